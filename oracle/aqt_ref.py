"""numpy restatement of aqt.jax.v2's quantized dot_general (test infrastructure).

Every function cites the reference lines it follows (paths relative to the
reference checkout, `aqt/jax/v2/...`).  Arrays are numpy float32; a dtype tag
('f32' or 'bf16') travels next to each float array and every op rounds its
result to the tag's format, which is what an eager (op-by-op) JAX run does.
Integer qvalues are int8 arrays (int4 values live in an int8 container, as the
reference's jnp.int4 does logically); fp8 qvalues are float32 arrays holding
fp8-representable values.
"""
from __future__ import annotations

import copy
import dataclasses
from typing import Any, Optional, Sequence

import numpy as np

from oracle import numerics as nm
from oracle import prng

F32, BF16 = nm.F32, nm.BF16
FP8 = ('e4m3', 'e5m2')

# When True the PRNG helpers use the `jax_threefry_partitionable=True` layout.
PARTITIONABLE = False


# ----------------------------------------------------------------------------
# Config mirrors (only the knobs that change arithmetic).


@dataclasses.dataclass
class QuantizerCfg:
  """aqt_quantizer.Quantizer + its numerics (aqt_quantizer.py:38-62)."""

  bits: Any = None  # None | int | 'e4m3' | 'e5m2'  (numerics/utils.py:22-48)
  noise: Optional[str] = None  # None | 'jax.uniform' | 'custom-1'
  noise_sharing_axes: Sequence[int] = ()
  fp8_sr: bool = False  # Fp8Numerics.stochastic_rounding
  calib_shared_axes: Any = None  # None | 'per_tensor' | sequence of axes
  scale_dtype: Optional[str] = None  # Calibration.dtype
  po2_scale: bool = False
  clipping_scale: Optional[float] = None
  const_bound: Optional[float] = None  # ConstantCalibration(bound=...)
  abs_mean_p: Optional[float] = None  # AbsMeanCalibration(p=..., clipping_scale=...)
  auto_clip_search: Optional[Sequence[float]] = None  # SnrBasedAutoCalibration
  preserve_zero: bool = True
  preserve_max_val: bool = False
  clip: bool = True
  round: bool = True
  keep_float: bool = False  # numerics.dtype = None: qvalue stays in the input dtype
  key: Optional[np.ndarray] = None  # Context.key
  # (full shape, per-axis index arrays): the tensor being quantized is the sub-block
  # full[np.ix_(*indices)] of a larger one and draws that tensor's noise at its own positions
  # (for checking slices of tensors too large to restate whole; 'jax.uniform' noise and the fp8
  # mantissa noise)
  noise_window: Any = None

  def is_int(self):
    return isinstance(self.bits, int)

  def is_fp8(self):
    return self.bits in FP8


@dataclasses.dataclass
class RawCfg:
  """aqt_dot_general.DotGeneralRaw (aqt_dot_general.py:732-749)."""

  lhs: QuantizerCfg
  rhs: QuantizerCfg
  rhs_use_fwd_quant: bool = False  # Tensor.use_fwd_quant of the rhs side
  lhs_dequant_mode: str = 'output'  # 'output' | 'this_input' | 'other_input'
  rhs_dequant_mode: str = 'output'
  lhs_calibration_mode: str = 'ca'  # 'ca' | 'ra'
  rhs_calibration_mode: str = 'ca'
  local_aqt_shard_count: Optional[int] = None
  acc: Any = 'auto'  # 'auto' follows dot_general_raw_make; None | 'i32' | 'f32'

  def accumulator(self):
    # aqt_dot_general.py:110-123 / config.py:117-137
    if self.acc != 'auto':
      return self.acc
    lb, rb = self.lhs.bits, self.rhs.bits
    if isinstance(lb, int) and isinstance(rb, int) and 2 <= lb <= 8 and 2 <= rb <= 8:
      return 'i32'
    if lb in FP8 and rb in FP8:
      return 'f32'
    return None


@dataclasses.dataclass
class DgCfg:
  fwd: RawCfg
  dlhs: RawCfg
  drhs: RawCfg


def dot_general_make(lhs_bits=None, rhs_bits=None, bwd_bits=None, use_fwd_quant=True):
  """aqt_dot_general.py:161-203."""
  cfg = DgCfg(
      fwd=RawCfg(QuantizerCfg(bits=lhs_bits), QuantizerCfg(bits=rhs_bits)),
      dlhs=RawCfg(QuantizerCfg(bits=bwd_bits), QuantizerCfg(bits=bwd_bits)),
      drhs=RawCfg(QuantizerCfg(bits=bwd_bits), QuantizerCfg(bits=bwd_bits)),
  )
  if lhs_bits is not None:
    cfg.drhs.rhs_use_fwd_quant = use_fwd_quant
  if rhs_bits is not None:
    cfg.dlhs.rhs_use_fwd_quant = use_fwd_quant
  return cfg


def set_stochastic_rounding(cfg, vjp_lhs, vjp_rhs, implementation='jax.uniform',
                            noise_sharing_axes=()):
  """config.py:171-225."""
  for raw in (cfg.dlhs, cfg.drhs):
    for q, on in ((raw.lhs, vjp_lhs), (raw.rhs, vjp_rhs)):
      if q.is_fp8():
        q.fp8_sr = bool(on)
      else:
        q.noise = implementation if on else None
        q.noise_sharing_axes = tuple(noise_sharing_axes)


def fully_quantized(fwd_bits=8, bwd_bits=8, use_fwd_quant=True,
                    use_stochastic_rounding=True):
  """config.py:598-658 (old-style SR switch only)."""
  cfg = dot_general_make(fwd_bits, fwd_bits, bwd_bits, use_fwd_quant)
  if use_stochastic_rounding:
    set_stochastic_rounding(cfg, True, True, 'jax.uniform')
  return cfg


def config_v4(fwd_bits=8, dlhs_bits=8, drhs_bits=None, rng_type='jax.uniform',
              dlhs_use_fwd_quant=None, drhs_use_fwd_quant=None):
  """config.py:724-788; set_bits forces use_fwd_quant False (config.py:505-511)."""
  cfg = DgCfg(
      fwd=RawCfg(QuantizerCfg(bits=fwd_bits), QuantizerCfg(bits=fwd_bits)),
      dlhs=RawCfg(QuantizerCfg(bits=dlhs_bits), QuantizerCfg(bits=dlhs_bits)),
      drhs=RawCfg(QuantizerCfg(bits=drhs_bits), QuantizerCfg(bits=drhs_bits)),
  )
  set_stochastic_rounding(cfg, True, False, rng_type)
  if dlhs_use_fwd_quant is not None:
    cfg.dlhs.rhs_use_fwd_quant = dlhs_use_fwd_quant
  if drhs_use_fwd_quant is not None:
    cfg.drhs.rhs_use_fwd_quant = drhs_use_fwd_quant
  return cfg


def set_context(cfg, key):
  """config.py:66-90: key -> (fwd, dlhs, drhs) -> (lhs, rhs) each."""
  cfg = copy.deepcopy(cfg)
  if key is None:
    return cfg
  k3 = prng.split(key, 3, PARTITIONABLE)
  for raw, k in zip((cfg.fwd, cfg.dlhs, cfg.drhs), k3):
    k2 = prng.split(k, 2, PARTITIONABLE)
    raw.lhs.key = k2[0]
    raw.rhs.key = k2[1]
  return cfg


# ----------------------------------------------------------------------------
# Numerics.


def int_quant_bound(q: QuantizerCfg):
  """int_numerics.py:51-64 (table :42-49)."""
  edge = 2.0 ** (q.bits - 1) - (0.5 if q.preserve_zero else 0.0)
  return edge - 0.5 if q.preserve_max_val else edge


def int_clip_bound(q: QuantizerCfg):
  """int_numerics.py:66-76."""
  edge = 2.0 ** (q.bits - 1) - (0.5 if q.preserve_zero else 0.0)
  return edge - 0.5 if q.round else edge


def quant_bound(q: QuantizerCfg):
  if q.is_fp8():
    # fp8_numerics.py:79-86: finfo(dtype).max as bf16 (both exact in bf16).
    return nm.E4M3_MAX if q.bits == 'e4m3' else nm.E5M2_MAX
  return int_quant_bound(q)


def _noise_shape(shape, sharing_axes):
  """stochastic_rounding.py:25-32."""
  return tuple(1 if ax in sharing_axes else s for ax, s in enumerate(shape))


def jax_uniform_noise(shape, key, sharing_axes=()):
  """stochastic_rounding.py:36-46: uniform(key, shape) - 0.5, float32."""
  ns = _noise_shape(shape, sharing_axes)
  return prng.uniform(key, ns, PARTITIONABLE) - np.float32(0.5)


def jax_uniform_noise_window(shape, key, window, kind='jax.uniform', sharing_axes=()):
  """jax_uniform_noise of the enclosing tensor, read at the positions of a sub-block."""
  assert kind == 'jax.uniform' and not sharing_axes
  total, flat = _window_flat_index(shape, window)
  return prng.uniform_at(key, total, flat, PARTITIONABLE) - np.float32(0.5)


def random_centered_uniform_noise(shape, key, sharing_axes=()):
  """stochastic_rounding.py:50-78 ('custom-1')."""
  ns = _noise_shape(shape, sharing_axes)
  bits = prng.random_bits(key, ns, 16, PARTITIONABLE).astype(np.uint32)
  pat = (bits << np.uint32(23 - 16)) | np.uint32(0x3F800000)
  floats = pat.view(np.float32)
  shift = np.float32(2.0 ** (-1 - 16))
  return floats - (np.float32(1.5) - shift)


def int_vjp_fwd(x, dt, q: QuantizerCfg):
  """IntSymmetric.vjp_fwd (int_numerics.py:81-111). Returns (values, dtype tag)."""
  assert q.bits <= 22
  if q.noise is not None:
    assert q.key is not None, 'noise_fn is set but no key in Context'
    fn = {'jax.uniform': jax_uniform_noise,
          'custom-1': random_centered_uniform_noise}[q.noise]
    if q.noise_window is not None:
      noise = jax_uniform_noise_window(x.shape, q.key, q.noise_window, q.noise, q.noise_sharing_axes)
    else:
      noise = fn(x.shape, q.key, q.noise_sharing_axes)
    # x (dt) + noise (f32) promotes to f32; one f32 rounding, then astype(dt).
    x = nm.cast(x.astype(np.float32) + noise, dt)
  if q.clip:
    b = np.float32(int_clip_bound(q))
    x = np.clip(x, -b, b)
  if q.round:
    if q.preserve_zero:
      x = np.rint(x)  # lax.round(TO_NEAREST_EVEN)
    else:
      x = nm.cast(np.floor(x) + np.float32(0.5), dt)
  if q.preserve_zero and 2 <= q.bits <= 8 and not q.keep_float:
    # numerics/utils.py:36-47 + utils.py:120-135: int4 for 4 bits, else int8.
    return x.astype(np.int8), ('i4' if q.bits == 4 else 'i8')
  return x.astype(np.float32), dt


def _window_flat_index(shape, window):
  full_shape, indices = window
  assert tuple(len(i) for i in indices) == tuple(shape)
  flat = np.ravel_multi_index(np.ix_(*[np.asarray(i, np.int64) for i in indices]), full_shape)
  return int(np.prod(full_shape, dtype=np.int64)), flat


def fp_mantissa_round(x, dt, mantissa_bits, key, window=None):
  """fp8_numerics.py:36-64: add masked random bits to the mantissa, truncate.  `window`: x is a
  sub-block of a larger tensor and takes that tensor's bits at its own positions."""
  assert dt in (BF16, F32)
  if dt == BF16:
    nmant, width = 7, 16
    u = nm.bf16_bits(x)
  else:
    nmant, width = 23, 32
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).copy()
  noise_bits = nmant - mantissa_bits
  mask = u.dtype.type((1 << noise_bits) - 1)
  if window is not None:
    total, flat = _window_flat_index(x.shape, window)
    noise = prng.random_bits_at(key, total, flat, PARTITIONABLE, width).astype(u.dtype) & mask
  else:
    noise = prng.random_bits(key, x.shape, width, PARTITIONABLE) & mask
  with np.errstate(over='ignore'):
    u = (u + noise) & ~mask
  return nm.from_bf16_bits(u) if dt == BF16 else u.view(np.float32)


def fp8_vjp_fwd(x, dt, q: QuantizerCfg):
  """Fp8Numerics.vjp_fwd (fp8_numerics.py:88-123)."""
  mant = 3 if q.bits == 'e4m3' else 2
  if q.fp8_sr:
    assert q.key is not None
    x = fp_mantissa_round(x, dt, mant, q.key, q.noise_window)
  b = np.float32(quant_bound(q))
  x = np.clip(x, -b, b)
  x = nm.to_e4m3fn(x) if q.bits == 'e4m3' else nm.to_e5m2(x)
  return x, q.bits


# ----------------------------------------------------------------------------
# Calibration and QTensor.


@dataclasses.dataclass
class QTensor:
  """aqt_tensor.QTensor (aqt_tensor.py:55-94) minus sparsity/tiling."""

  qvalue: Optional[np.ndarray]
  qdtype: Optional[str]  # 'i8' | 'i4' | 'e4m3' | 'e5m2' | 'i32' | 'f32' | 'bf16'
  scale: list  # list of float32 arrays
  scale_dtype: Optional[str]
  dequant_dtype: str
  bias: list = dataclasses.field(default_factory=list)
  # dtype of each scale when they differ (a bf16 activation scale next to an f32 weight scale in
  # serving); None = all scales have scale_dtype.
  scale_dtypes: Optional[list] = None


def ceil_to_po2(scale, dt):
  """calibration.py:25-30, op by op in dtype `dt`."""
  r = nm.cast(np.float32(1.0) / scale, dt)
  l = nm.cast(np.log2(r), dt)
  p = nm.cast(np.exp2(np.floor(l)), dt)
  return nm.cast(np.float32(1.0) / p, dt)


def calibrate(x, dt, shared_axes, q: QuantizerCfg):
  """AbsMaxCalibration / ConstantCalibration / AbsMeanCalibration / SnrBasedAutoCalibration
  (calibration.py:68-399).

  Returns (scale float32 array with keepdims shape, scale dtype tag).
  """
  sdt = q.scale_dtype or dt
  axes = tuple(shared_axes)
  if q.auto_clip_search is not None:
    return _snr_calibrate(x, dt, axes, q), sdt
  qb = nm.cast(np.float32(quant_bound(q)), dt)
  if q.const_bound is not None:
    shape = [1 if a in axes else s for a, s in enumerate(x.shape)]
    bound = nm.cast(np.ones(shape, np.float32) * np.float32(q.const_bound), dt)
  elif q.abs_mean_p is not None:
    # calibration.py:160-193; sums accumulate in float32 and round once to dt (the order of
    # the summation inside XLA is not restated: parity unpinned for non-exact sums)
    p = nm.cast(np.float32(q.abs_mean_p), dt)
    powed = np.abs(x) if q.abs_mean_p == 1.0 else nm.cast(np.power(np.abs(x), p), dt)
    abs_sum = nm.cast(np.sum(powed.astype(np.float32), axis=axes, keepdims=True), dt)
    count = np.sum(x != 0.0, axis=axes, keepdims=True).astype(np.float32)
    count = np.where(count == 0.0, np.float32(1.0), count)
    mean = nm.cast(abs_sum / nm.cast(count, dt), dt)
    inv_p = nm.cast(np.float32(1.0 / q.abs_mean_p), dt)
    abs_mean = mean if q.abs_mean_p == 1.0 else nm.cast(np.power(mean, inv_p), dt)
    abs_mean = nm.cast(abs_mean * nm.cast(np.float32(q.clipping_scale), dt), dt)
    bound = np.where(abs_mean == 0.0, np.float32(1.0), abs_mean)
  else:
    abs_max = np.max(np.abs(x), axis=axes, keepdims=True).astype(np.float32)
    abs_max = np.where(abs_max == 0.0, np.float32(1.0), abs_max)
    if q.clipping_scale:
      bound = nm.cast(abs_max * nm.cast(np.float32(q.clipping_scale), dt), dt)
    else:
      bound = abs_max
  scale = nm.cast(bound / qb, dt)
  if q.po2_scale:
    scale = ceil_to_po2(scale, dt)
  return nm.cast(scale, sdt), sdt


def _snr_calibrate(x, dt, axes, q: QuantizerCfg):
  """SnrBasedAutoCalibration (calibration.py:196-399): for every candidate clipping scale the
  tensor is fake-quantized and log(1 + signal / noise) computed per group; the best candidate
  per group gives the scale.  The search keeps float32 state; the candidate scales are
  computed in the input dtype, the final one in float32 (abs_max * float32 clip)."""
  sdt = q.scale_dtype or dt
  x = np.asarray(x, np.float32)
  abs_max = np.max(np.abs(x), axis=axes, keepdims=True).astype(np.float32)
  abs_max = np.where(abs_max == 0.0, np.float32(1.0), abs_max)
  best = np.ones(abs_max.shape, np.float32)
  max_snr = np.zeros(abs_max.shape, np.float32)
  qbf = np.float32(quant_bound(q))
  for clip in q.auto_clip_search:
    # abs_max (dt) * python float stays in dt
    bound = nm.cast(abs_max * nm.cast(np.float32(clip), dt), dt)
    scale = nm.cast(nm.cast(bound / nm.cast(qbf, dt), dt), sdt)
    qt = calculate_qvalue(x, dt, QTensor(None, None, [scale], sdt, dt), q)
    err = nm.cast(x - dequant(qt), dt)
    noise = nm.cast(np.sum(nm.cast(err * err, dt).astype(np.float32), axis=axes, keepdims=True), dt)
    signal = nm.cast(np.sum(nm.cast(x * x, dt).astype(np.float32), axis=axes, keepdims=True), dt)
    with np.errstate(divide='ignore', invalid='ignore'):
      ratio = nm.cast(signal / noise, dt)
      snr = nm.cast(np.log(nm.cast(np.float32(1.0) + ratio, dt)), dt)
    better = snr > max_snr
    best = np.where(better, np.float32(clip), best)
    max_snr = np.maximum(snr, max_snr)
  bound = abs_max * best  # float32: dt array times a float32 array
  scale = bound / qbf
  if q.po2_scale:
    scale = ceil_to_po2(scale, 'f32')
  return nm.cast(scale, sdt)


def qtensor_quant(x, dt, scales, sdt):
  """QTensor.quant (aqt_tensor.py:125-159): multiply by the reciprocal scale."""
  qv, qdt = x, dt
  for s in scales:
    s_inv = nm.cast(np.float32(1.0) / s, sdt)
    s_inv = np.where(np.isinf(s_inv), np.float32(1.0), s_inv)
    qdt = nm.promote(qdt, sdt)
    qv = nm.cast(qv * s_inv, qdt)
  return qv, qdt


def quantize(x, dt, q: QuantizerCfg, calibration_axes):
  """Quantizer.quant = calibrate + calculate_qvalue (aqt_quantizer.py:65-176)."""
  x = np.asarray(x, np.float32)
  if q.bits is None:
    # NoNumerics bypass (aqt_quantizer.py:111-120,163-164).
    return QTensor(x, dt, [], None, dt)
  if q.calib_shared_axes == 'per_tensor':
    shared = list(range(x.ndim))
  else:
    shared = q.calib_shared_axes or calibration_axes
  scale, sdt = calibrate(x, dt, shared, q)
  return calculate_qvalue(x, dt, QTensor(None, None, [scale], sdt, dt), q)


def calculate_qvalue(x, dt, qt: QTensor, q: QuantizerCfg):
  """Quantizer.calculate_qvalue (aqt_quantizer.py:159-176)."""
  if q.bits is None:
    return qt
  v, vdt = qtensor_quant(np.asarray(x, np.float32), dt, qt.scale, qt.scale_dtype)
  if q.is_fp8():
    qv, qdt = fp8_vjp_fwd(v, vdt, q)
  else:
    qv, qdt = int_vjp_fwd(v, vdt, q)
  return QTensor(qv, qdt, list(qt.scale), qt.scale_dtype, qt.dequant_dtype)


def dequant(qt: QTensor):
  """QTensor.dequant (aqt_tensor.py:161-200): cast first, then scales in order."""
  dd = qt.dequant_dtype
  if qt.qdtype in ('i8', 'i4', 'i32'):
    ret = nm.int32_to_float(qt.qvalue, dd)
  else:
    ret = nm.cast(qt.qvalue, dd)
  rdt = dd
  for i, s in enumerate(qt.scale):
    sdt = qt.scale_dtypes[i] if qt.scale_dtypes else (qt.scale_dtype or dd)
    rdt = nm.promote(rdt, sdt)  # jnp promotion of `ret * scale`, product by product
    ret = nm.cast(ret * s, rdt)
  return nm.cast(ret, dd)


# ----------------------------------------------------------------------------
# Scale re-layout (transpose.py).


def get_remaining_axes(rank, ca, ba):
  """utils.py:138-148."""
  return [i for i in range(rank) if i not in list(ca) + list(ba)]


def _scale_trans(x, ca, ba):
  """transpose.py:98-111."""
  ca, ba = list(ca), list(ba)
  for i in ca:
    assert x.shape[i] == 1
  ra = get_remaining_axes(x.ndim, ca, ba)
  x = np.transpose(x, ba + ra + ca)
  return x.reshape(x.shape[: len(ba) + len(ra)])


def lhs_scale_transpose_to_output(s, dn, lhs_shape, rhs_shape):
  """transpose.py:114-132."""
  (lca, rca), (lba, rba) = dn
  t = _scale_trans(s, lca, lba)
  n_rhs_ra = len(rhs_shape) - len(rca) - len(rba)
  return t.reshape(t.shape + (1,) * n_rhs_ra)


def rhs_scale_transpose_to_output(s, dn, lhs_shape, rhs_shape):
  """transpose.py:135-148."""
  (lca, rca), (lba, rba) = dn
  t = _scale_trans(s, rca, rba)
  n_lhs_ra = len(lhs_shape) - len(lca) - len(lba)
  nb = len(rba)
  return t.reshape(t.shape[:nb] + (1,) * n_lhs_ra + t.shape[nb:])


def _scale_trans_for_other_input(x, my_ca, my_ba, other_ca, other_ba, other_rank):
  """transpose.py:218-263."""
  my_ca, my_ba = list(my_ca), list(my_ba)
  other_ca, other_ba = list(other_ca), list(other_ba)
  if x.ndim < other_rank:
    x = x.reshape(list(x.shape) + [1] * (other_rank - x.ndim))
  perm = [-1] * x.ndim
  my_ra = get_remaining_axes(x.ndim, my_ca, my_ba)
  for a in my_ra:
    assert x.shape[a] == 1
  for mine, other in zip(my_ca + my_ba, other_ca + other_ba):
    perm[other] = mine
  it = iter(my_ra)
  perm = [next(it) if p == -1 else p for p in perm]
  x = np.transpose(x, perm)
  if x.ndim > other_rank:
    x = x.reshape(x.shape[:other_rank])
  return x


def rhs_scale_transpose_for_lhs_input(s, dn, lhs_shape):
  (lca, rca), (lba, rba) = dn
  return _scale_trans_for_other_input(s, rca, rba, lca, lba, len(lhs_shape))


def lhs_scale_transpose_for_rhs_input(s, dn, rhs_shape):
  (lca, rca), (lba, rba) = dn
  return _scale_trans_for_other_input(s, lca, lba, rca, rba, len(rhs_shape))


# ----------------------------------------------------------------------------
# dot_general.


def lax_dot_general(lhs, rhs, dn, out_np_dtype):
  """lax.dot_general on numpy arrays; exact (float64 accumulate, then cast).

  Output axis order: batch, lhs remaining, rhs remaining.  Products of
  int8/fp8/bf16 values and sums of up to 2**20 of them are exact in float64 for
  the integer case; for floats the float64 result is rounded once.
  """
  (lca, rca), (lba, rba) = dn
  lca, rca, lba, rba = list(lca), list(rca), list(lba), list(rba)
  lra = get_remaining_axes(lhs.ndim, lca, lba)
  rra = get_remaining_axes(rhs.ndim, rca, rba)
  lt = np.transpose(lhs, lba + lra + lca).astype(np.float64)
  rt = np.transpose(rhs, rba + rca + rra).astype(np.float64)
  bshape = lt.shape[: len(lba)]
  mshape = lt.shape[len(lba): len(lba) + len(lra)]
  kshape = lt.shape[len(lba) + len(lra):]
  nshape = rt.shape[len(rba) + len(rca):]
  b = int(np.prod(bshape, dtype=np.int64))
  m = int(np.prod(mshape, dtype=np.int64))
  k = int(np.prod(kshape, dtype=np.int64))
  n = int(np.prod(nshape, dtype=np.int64))
  out = np.matmul(lt.reshape(b, m, k), rt.reshape(b, k, n))
  out = out.reshape(bshape + mshape + nshape)
  if np.issubdtype(out_np_dtype, np.integer):
    return np.rint(out).astype(out_np_dtype)
  return out.astype(out_np_dtype)


def qtensor_dot_general(lhs_qt: QTensor, rhs_qt: QTensor, dn, raw: RawCfg, dequant_dtype):
  """_qtensor_dot_general (aqt_dot_general.py:843-958)."""

  def maybe_dequant(qt, mode):
    if mode == 'this_input':
      return dequant(qt), qt.dequant_dtype
    return qt.qvalue, qt.qdtype

  lq, ldt = maybe_dequant(lhs_qt, raw.lhs_dequant_mode)
  rq, rdt = maybe_dequant(rhs_qt, raw.rhs_dequant_mode)
  if raw.lhs_dequant_mode == 'other_input':
    assert rdt in (F32, BF16)
    for s in lhs_qt.scale:
      t = lhs_scale_transpose_for_rhs_input(s, dn, rq.shape)
      rq = nm.cast(rq * nm.cast(t, rdt), rdt)
  if raw.rhs_dequant_mode == 'other_input':
    assert ldt in (F32, BF16)
    for s in rhs_qt.scale:
      t = rhs_scale_transpose_for_lhs_input(s, dn, lq.shape)
      lq = nm.cast(lq * nm.cast(t, ldt), ldt)

  # cfg.dot_general(..., preferred_element_type=dg_accumulator_dtype)
  # (aqt_dot_general.py:921-927).  With None the result takes the promoted
  # operand dtype (integer containers promote to the float operand's dtype).
  acc = raw.accumulator()
  ints = ('i8', 'i4')
  if acc == 'i32':
    assert ldt in ints and rdt in ints, (ldt, rdt)  # aqt_dot_general.py:876-880
    out, odt = lax_dot_general(lq, rq, dn, np.int32), 'i32'
  else:
    if acc == 'f32':
      odt = F32
    else:
      fl = [d for d in (ldt, rdt) if d in (F32, BF16)]
      assert fl, 'integer x integer without an int32 accumulator is not restated'
      odt = F32 if F32 in fl else BF16
    out = nm.cast(lax_dot_general(lq, rq, dn, np.float32), odt)

  # Each scale keeps its own dtype: dequant multiplies them in one by one and jnp promotes
  # product by product (a bf16 lhs scale next to an f32 rhs scale rounds the first product only).
  scales, sdts = [], []
  if raw.lhs_dequant_mode == 'output':
    for i, s in enumerate(lhs_qt.scale):
      scales.append(lhs_scale_transpose_to_output(s, dn, lq.shape, rq.shape))
      sdts.append(lhs_qt.scale_dtypes[i] if lhs_qt.scale_dtypes else (lhs_qt.scale_dtype or dequant_dtype))
  if raw.rhs_dequant_mode == 'output':
    for i, s in enumerate(rhs_qt.scale):
      scales.append(rhs_scale_transpose_to_output(s, dn, lq.shape, rq.shape))
      sdts.append(rhs_qt.scale_dtypes[i] if rhs_qt.scale_dtypes else (rhs_qt.scale_dtype or dequant_dtype))
  return QTensor(out, odt, scales, None, dequant_dtype, scale_dtypes=sdts or None)


def _apply_local_aqt(shard_count, lhs, rhs, dn):
  """_apply_local_aqt, factor_reshape variant (aqt_dot_general.py:302-328)."""

  def factor(x, ca, ba):
    ca, ba = list(ca), list(ba)
    if not ca:
      return x, ca, ba
    shape = list(x.shape)
    ax = ca[0]
    assert shape[ax] % shard_count == 0
    size = shape[ax] // shard_count
    shape[ax] = shard_count
    shape.insert(ax + 1, size)
    new_ca = [b + int(b >= ax) for b in ca]
    new_ba = [ax] + [b + int(b > ax) for b in ba]
    return x.reshape(shape), new_ca, new_ba

  (lca, rca), (lba, rba) = dn
  lhs, lca, lba = factor(lhs, lca, lba)
  rhs, rca, rba = factor(rhs, rca, rba)
  return lhs, rhs, ((lca, rca), (lba, rba))


def _sum_leading(x):
  """jnp.sum(x, axis=0): float32 accumulation in index order, one final cast."""
  acc = np.zeros(x.shape[1:], np.float32)
  for i in range(x.shape[0]):
    acc = acc + x[i]
  return acc


@dataclasses.dataclass
class Residual:
  """MultiTensor (aqt_dot_general.py:209-213)."""

  x: np.ndarray
  dt: str
  qx: QTensor


def dg_raw(lhs, ldt, rhs, rdt, dn, raw: RawCfg, lhs_qt=None, rhs_qt=None):
  """DotGeneralRaw.__call__ (aqt_dot_general.py:757-840).

  `rhs` may be a Residual (the bwd calls pass the fwd residual).
  Returns (out float32 array, out dtype tag, (lhs Residual, rhs Residual), acc QTensor).
  """
  if isinstance(rhs, Residual):
    # _maybe_use_fwd_quant (aqt_dot_general.py:675-729)
    res = rhs
    if raw.rhs_use_fwd_quant:
      assert len(res.qx.scale) == 1 and not res.qx.bias
      t = rhs_scale_transpose_for_lhs_input(res.qx.scale[0], dn, lhs.shape)
      lhs = nm.cast(lhs * nm.cast(t, ldt), ldt)
      rdt = res.qx.dequant_dtype
      rhs = nm.cast(np.asarray(res.qx.qvalue, np.float32), rdt)
    else:
      rhs, rdt = res.x, res.dt
  lhs = np.asarray(lhs, np.float32)
  rhs = np.asarray(rhs, np.float32)

  if raw.local_aqt_shard_count is not None:
    lhs, rhs, dn = _apply_local_aqt(raw.local_aqt_shard_count, lhs, rhs, dn)

  (lca, rca), (lba, rba) = dn

  def calib_axes(mode, ndim, ca, ba):
    return get_remaining_axes(ndim, ca, ba) if mode == 'ra' else list(ca)

  # quant() (aqt_dot_general.py:598-672): a provided full QTensor replaces the
  # computed one; a scale-only one supplies the scale.
  def side(x, dt, q, mode, ca, ba, given):
    if given is not None and given.qvalue is not None:
      return given
    if given is not None:
      return calculate_qvalue(x, dt, given, q)
    return quantize(x, dt, q, calib_axes(mode, x.ndim, ca, ba))

  lqt = side(lhs, ldt, raw.lhs, raw.lhs_calibration_mode, lca, lba, lhs_qt)
  rqt = side(rhs, rdt, raw.rhs, raw.rhs_calibration_mode, rca, rba, rhs_qt)

  dd = nm.promote(ldt, rdt)
  acc_qt = qtensor_dot_general(lqt, rqt, dn, raw, dd)
  out = dequant(acc_qt)
  if raw.local_aqt_shard_count is not None and len(lca) > 0:
    # aqt_dot_general.py:832-837: sum of the per-shard dequantized outputs.
    out = nm.cast(_sum_leading(out), dd)
  return out, dd, (Residual(lhs, ldt, lqt), Residual(rhs, rdt, rqt)), acc_qt


def bwd_dimension_numbers(fwd_dn, y_is_lhs, gradient_rank, y_rank):
  """_update_dimension_numbers_for_backward (aqt_dot_general.py:1127-1175)."""

  def ranges_like(*xs):
    start = 0
    for x in xs:
      yield tuple(range(start, start + len(x)))
      start += len(x)

  (x_ca, y_ca), (x_ba, y_ba) = fwd_dn
  if y_is_lhs:
    (y_ca, x_ca) = (x_ca, y_ca)
    (y_ba, x_ba) = (x_ba, y_ba)
  g_rank = gradient_rank - y_rank + len(x_ba) + 2 * len(x_ca)
  x_ra = tuple(get_remaining_axes(g_rank, x_ca, x_ba))
  y_ra = tuple(get_remaining_axes(y_rank, y_ca, y_ba))
  if y_is_lhs:
    g_ba, g_ca, _ = ranges_like(x_ba, y_ra, x_ra)
  else:
    g_ba, _, g_ca = ranges_like(x_ba, x_ra, y_ra)
  dims = ((g_ca, y_ra), (g_ba, tuple(y_ba)))
  x_ca_sorted_by_y = tuple(np.take(x_ca, np.argsort(y_ca)).tolist())
  out_axes = tuple(np.argsort(tuple(x_ba) + x_ra + x_ca_sorted_by_y).tolist())
  return dims, out_axes


@dataclasses.dataclass
class FwdResult:
  out: np.ndarray
  out_dtype: str
  lhs_res: Residual
  rhs_res: Residual
  acc: QTensor


def dg_fwd(lhs, rhs, dt, dn, cfg: DgCfg, lhs_qt=None, rhs_qt=None) -> FwdResult:
  """dg_core_vjp_fwd (aqt_dot_general.py:1098-1124); lhs/rhs share dtype `dt`."""
  lhs = nm.cast(lhs, dt)
  rhs = nm.cast(rhs, dt)
  out, odt, (lres, rres), acc = dg_raw(lhs, dt, rhs, dt, dn, cfg.fwd, lhs_qt, rhs_qt)
  return FwdResult(nm.cast(out, dt), dt, lres, rres, acc)


def dg_bwd(g, gdt, dn, fwd: FwdResult, cfg: DgCfg, return_acc=False):
  """dg_core_vjp_bwd (aqt_dot_general.py:1178-1221). Returns (dlhs, drhs)."""
  g = nm.cast(g, gdt)
  outs, accs = [], []
  for y_res, raw, y_is_lhs in ((fwd.rhs_res, cfg.dlhs, False), (fwd.lhs_res, cfg.drhs, True)):
    dims, out_axes = bwd_dimension_numbers(dn, y_is_lhs, g.ndim, y_res.x.ndim)
    out, odt, _, acc = dg_raw(g, gdt, y_res, None, dims, raw)
    outs.append(np.transpose(out, out_axes))
    accs.append(acc)
  if return_acc:
    return outs[0], outs[1], accs
  return outs[0], outs[1]


# ----------------------------------------------------------------------------
# Subchannel (tiled) dot_general for a contraction-axis tiling
# (tiled_dot_general.py:401-543 restricted to contraction-axis tiles).


def tiled_dg_fwd(lhs, rhs, dt, tile_size, cfg: DgCfg):
  """Matmul [M,K]x[K,N] with the contraction axis split in tiles of tile_size.

  tiled_dot_general.py:430-435 makes the tile-count axis a leading batch axis of
  the inner dot_general; :493 sums the dequantized per-tile outputs.
  """
  m, k = lhs.shape
  k2, n = rhs.shape
  assert k == k2 and k % tile_size == 0
  t = k // tile_size
  lt = nm.cast(lhs, dt).reshape(m, t, tile_size)
  rt = nm.cast(rhs, dt).reshape(t, tile_size, n)
  dn = (((2,), (1,)), ((1,), (0,)))
  res = dg_fwd(lt, rt, dt, dn, cfg)  # out [t, m, n]
  # jnp.sum over the tile axis in dtype dt: XLA accumulates bf16 sums in f32
  # and rounds once at the end.
  return nm.cast(_sum_leading(res.out), dt), res


# ----------------------------------------------------------------------------
# ragged_dot (aqt_ragged_dot.py:49-86): forward only.


def lax_ragged_dot(lhs, rhs, group_sizes, out_np_dtype):
  """jax.lax.ragged_dot: consecutive row groups of lhs [m, k] times rhs[g] [k, n]."""
  m, n = lhs.shape[0], rhs.shape[2]
  out = np.zeros((m, n), np.float64)
  start = 0
  for g, size in enumerate(group_sizes):
    size = int(size)
    out[start:start + size] = lhs[start:start + size].astype(np.float64) @ rhs[g].astype(np.float64)
    start += size
  if np.issubdtype(out_np_dtype, np.integer):
    return np.rint(out).astype(out_np_dtype)
  return out.astype(out_np_dtype)


def ragged_dot_fwd(lhs, rhs, dt, group_sizes, raw: RawCfg):
  """The fwd DotGeneralRaw with `dot_general = RaggedDot(group_sizes)` and
  dimension_numbers ([1], [0, 1]), ([], []): the rhs scale is shared by all groups."""
  dn = (((1,), (0, 1)), ((), ()))
  lhs, rhs = nm.cast(lhs, dt), nm.cast(rhs, dt)
  lqt = quantize(lhs, dt, raw.lhs, [1])
  rqt = quantize(rhs, dt, raw.rhs, [0, 1])
  acc = raw.accumulator()
  if acc == 'i32':
    out, odt = lax_ragged_dot(lqt.qvalue, rqt.qvalue, group_sizes, np.int32), 'i32'
  else:
    out, odt = nm.cast(lax_ragged_dot(lqt.qvalue, rqt.qvalue, group_sizes, np.float32), dt), dt
  scales, sdts = [], []
  for s in lqt.scale:
    scales.append(lhs_scale_transpose_to_output(s, dn, lhs.shape, rhs.shape))
    sdts.append(lqt.scale_dtype or dt)
  for s in rqt.scale:
    scales.append(rhs_scale_transpose_to_output(s, dn, lhs.shape, rhs.shape))
    sdts.append(rqt.scale_dtype or dt)
  return nm.cast(dequant(QTensor(out, odt, scales, None, dt, scale_dtypes=sdts or None)), dt), lqt, rqt


# ----------------------------------------------------------------------------
# conv_general_dilated (aqt_conv_general.py:33-135), Flax layout, forward.


def lax_conv_nhwc(lhs, rhs, strides, padding, rhs_dilation=None):
  """jax.lax.conv_general_dilated for input N...C, kernel ...IO, output N...C in float64 (exact
  for the integer-valued operands it is used on here)."""
  ns = lhs.ndim - 2
  dil = list(rhs_dilation) if rhs_dilation is not None else [1] * ns
  kernel = rhs.shape[:ns]
  eff = [(k - 1) * d + 1 for k, d in zip(kernel, dil)]
  if isinstance(padding, str):
    pads = []
    for size, k, s in zip(lhs.shape[1:1 + ns], eff, strides):
      if padding.upper() == 'VALID':
        pads.append((0, 0))
      else:
        out = -(-size // s)
        total = max((out - 1) * s + k - size, 0)
        pads.append((total // 2, total - total // 2))
  else:
    pads = [tuple(p) for p in padding]
  x = np.pad(lhs.astype(np.float64), [(0, 0)] + pads + [(0, 0)])
  out_sizes = [(x.shape[1 + d] - eff[d]) // strides[d] + 1 for d in range(ns)]
  out = np.zeros([lhs.shape[0]] + out_sizes + [rhs.shape[-1]], np.float64)
  for tap in np.ndindex(*kernel):
    sl = [slice(None)]
    for d in range(ns):
      start = tap[d] * dil[d]
      sl.append(slice(start, start + (out_sizes[d] - 1) * strides[d] + 1, strides[d]))
    out += np.tensordot(x[tuple(sl)], rhs[tap].astype(np.float64), axes=([-1], [0]))
  return out


def conv_general_dilated_fwd(lhs, rhs, dt, strides, padding, raw: RawCfg, rhs_dilation=None):
  """The input shares a scale over all axes but the batch axis, the kernel over all but the
  output features (aqt_conv_general.py:203-226); the convolution runs on the quantized values
  held in the float dtype, the result is multiplied by the lhs scale, then the rhs scale."""
  lhs, rhs = nm.cast(lhs, dt), nm.cast(rhs, dt)
  rank = lhs.ndim
  lq = copy.copy(raw.lhs)
  lq.calib_shared_axes = list(range(1, rank))
  rq = copy.copy(raw.rhs)
  rq.calib_shared_axes = list(range(0, rank - 1))
  lqt = quantize(lhs, dt, lq, None)
  rqt = quantize(rhs, dt, rq, None)
  acc = nm.cast(lax_conv_nhwc(np.asarray(lqt.qvalue, np.float32), np.asarray(rqt.qvalue, np.float32), strides,
                              padding, rhs_dilation).astype(np.float32), dt)
  sdts = [lqt.scale_dtype or dt] * len(lqt.scale) + [rqt.scale_dtype or dt] * len(rqt.scale)
  out = dequant(QTensor(acc, dt, list(lqt.scale) + list(rqt.scale), None, dt, scale_dtypes=sdts or None))
  return nm.cast(out, dt), lqt, rqt

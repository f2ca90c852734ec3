"""Helpers shared by the GPU parity tests (numpy <-> torch, oracle adapters)."""
import numpy as np
import torch

from aqt_amd import _lib as L
from oracle import aqt_ref as R
from oracle import numerics as nm

TORCH_DT = {'f32': torch.float32, 'bf16': torch.bfloat16}


def to_dev(x, dt, dev):
  """float32 numpy (already representable in dt) -> torch tensor of dtype dt on dev."""
  return torch.from_numpy(np.ascontiguousarray(x, np.float32)).to(TORCH_DT[dt]).to(dev)


def rand(shape, dt, seed, scale=1.0, outliers=False):
  rng = np.random.default_rng(seed)
  x = rng.standard_normal(shape).astype(np.float32) * np.float32(scale)
  if outliers:
    mask = rng.random(shape) < 0.005
    x = np.where(mask, x * np.float32(20.0), x)
  return nm.cast(x, dt)


def fp8_bytes_to_float(b, kind):
  t = torch.from_numpy(np.ascontiguousarray(b, np.uint8))
  td = torch.float8_e4m3fn if kind == 'e4m3' else torch.float8_e5m2
  return t.view(td).float().numpy()


OUT_DT = {8: L.I8, 4: L.I4, 'e4m3': L.E4M3, 'e5m2': L.E5M2}
NOISE = {None: L.NOISE_NONE, 'jax.uniform': L.NOISE_JAX_UNIFORM, 'custom-1': L.NOISE_CUSTOM1}


def bounds(q: R.QuantizerCfg):
  if q.is_fp8():
    b = R.quant_bound(q)
    return b, b
  return R.int_quant_bound(q), R.int_clip_bound(q)

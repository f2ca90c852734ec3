"""Shared helpers and small types (mirrors aqt/jax/v2/utils.py:63-155).

The reference builds its configs from `flax.struct` dataclasses (mutable, slotted,
keyword-only).  Here they are plain mutable keyword-only dataclasses; "static"
and "dynamic" fields are the same thing because nothing is traced.
"""
from __future__ import annotations

import copy
import dataclasses
import enum
from typing import Any, Callable, Optional, Sequence, Union

import numpy as np
import torch

AxisIdx = int
AxisSize = int
# lax.dot_general-like callables: (lhs, rhs, dimension_numbers, precision=None,
# preferred_element_type=None) -> array.
DotGeneralT = Callable[..., Any]

dataclass = dataclasses.dataclass
flax_slots_dataclass = dataclasses.dataclass
flax_slots_kw_only_dataclass = lambda cls: dataclasses.dataclass(cls, kw_only=True)  # noqa: E731


def static_field(**kwargs):
  return dataclasses.field(**kwargs)


def dynamic_field(**kwargs):
  return dataclasses.field(**kwargs)


class _Int4:
  """Stands for jnp.int4: 4-bit values kept one per byte in an int8 tensor."""

  def __repr__(self):
    return 'torch.int4'  # printed like the torch dtypes it sits next to in configuration trees

  # One object stands for the dtype: configurations are deep-copied (set_context), and
  # `dtype is utils.int4` must keep holding for the copies.
  def __copy__(self):
    return self

  def __deepcopy__(self, memo):
    return self

  def __reduce__(self):
    return (_int4_singleton, ())


def _int4_singleton():
  return int4


# dtype names the reference takes from jax.numpy
int4 = _Int4()
int8 = torch.int8
int16 = torch.int16
int32 = torch.int32
bfloat16 = torch.bfloat16
float32 = torch.float32
float16 = torch.float16
float8_e4m3fn = torch.float8_e4m3fn
float8_e5m2 = torch.float8_e5m2


def assert_shape(shape, shape_template, msg: str):
  """A None entry of the template matches any extent (utils.py:48-55)."""
  shape, shape_template = list(shape), list(shape_template)
  assert len(shape) == len(shape_template), msg
  for got, want in zip(shape, shape_template):
    assert want is None or got == want, f'{msg}: {shape} does not match {shape_template}'


def assert_eq(value, expected, value_name: str):
  assert value == expected, f'{value_name}={value}, {expected=}'


class QuantMode(enum.Enum):
  """utils.py:85-89."""
  TRAIN = 1
  CALIBRATE = 2
  CONVERT = 3
  SERVE = 4


def infer_dtype_from_bits(bits: int):
  """utils.py:120-135."""
  if bits == 4:
    return int4
  if 2 <= bits <= 8:
    return int8
  return None


def get_remaining_axes(rank: int, contraction_axes: Sequence[int], batch_axes: Sequence[int]):
  """utils.py:138-148."""
  used = list(contraction_axes) + list(batch_axes)
  return [i for i in range(rank) if i not in used]


@dataclasses.dataclass
class Context:
  """utils.py:151-155. `key` is raw threefry key data: uint32[2], numpy, or a 2-word device tensor
  (read by the kernels where it lies: a key that changes between replays of a recorded step)."""
  key: Any = None
  train_step: Optional[int] = None
  quant_mode: QuantMode = QuantMode.TRAIN

  def __deepcopy__(self, memo):
    out = clone_fields(self)
    memo[id(self)] = out
    if out.key is not None and not isinstance(out.key, torch.Tensor):
      out.key = copy.deepcopy(self.key, memo)  # (a key in a device tensor is a handle: shared)
    return out


def clone_fields(obj):
  """A new object of obj's class holding the same field values (what copy.copy gives for a plain
  dataclass instance, without the pickle protocol round trip that makes it ~20x slower)."""
  fields = getattr(obj, '__dict__', None)
  if fields is None or hasattr(type(obj), '__slots__'):
    return copy.copy(obj)
  out = object.__new__(type(obj))
  out.__dict__.update(fields)
  return out


def deepcopy_fields(obj, memo, shared=()):
  """Deep copy of a plain config object: a new object of the same class whose fields are deep copies,
  except the ones named in `shared`, whose values are immutable (flags, numbers, enum members, dtype
  tags, functions) and stay shared.  Same result as copy.deepcopy's generic path at a fraction of its
  cost; configurations are copied on every layer call.  Fields a subclass adds are deep-copied."""
  out = clone_fields(obj)
  memo[id(obj)] = out
  d = out.__dict__
  for name, value in d.items():
    if name not in shared and value is not None:
      d[name] = copy.deepcopy(value, memo)
  return out


# Process-wide switch standing for jax.config.jax_threefry_partitionable: it selects
# which of the two jax.random counter layouts the noise kernels reproduce.
threefry_partitionable = False


def prng_key(seed: int) -> np.ndarray:
  """jax.random.PRNGKey(seed) as raw key data."""
  seed = int(seed) & 0xFFFFFFFFFFFFFFFF
  return np.array([seed >> 32, seed & 0xFFFFFFFF], dtype=np.uint32)

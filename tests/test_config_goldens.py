"""The configuration trees against the goldens the reference's own test holds
(aqt/jax/v2/config_test.py:44-648): every class name, field name, field order and default of
config_v4(<custom arguments>), config_v4() and config_fwd_fp8() after init_calibration() on the six
quantizers, compared as printed by pprint.

The golden texts (tests/golden/*.pprint.txt) are copied out of the reference's test as data by
tests/golden/make_config_goldens.py.  Three kinds of leaves print differently here than under
JAX and are mapped before the comparison, nothing else is: dtype objects
(<class 'jax.numpy.int8'> is torch.int8 here), the package path in class reprs
(aqt.jax.v2 -> aqt_amd.v2) and the default contraction hook (<function dot_general> is
lax_dot_general here).  Indentation depends on the width of those leaves, so both texts are
compared with all whitespace removed.
"""
import os
import pprint
import re

import pytest
import torch

from aqt_amd.v2 import config
from aqt_amd.v2 import utils

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden')


def _golden(name):
  with open(os.path.join(GOLDEN, f'{name}.pprint.txt')) as f:
    return f.read()


def _normalise_golden(s):
  s = re.sub(r"<class 'jax\.numpy\.(\w+)'>", lambda m: f'torch.{m.group(1)}', s)
  s = s.replace("'aqt.jax.v2.", "'aqt_amd.v2.")
  s = s.replace('<function dot_general>', '<function lax_dot_general>')
  return re.sub(r'\s+', '', s)


def _normalise_actual(s):
  s = re.sub(r' at 0x[0-9a-f]+>', '>', s)  # the reference's test removes memory addresses too
  return re.sub(r'\s+', '', s)


def _init_all_calibrations(cfg):
  # config_test.py:22-29
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    raw.dg_quantizer.lhs.init_calibration()
    raw.dg_quantizer.rhs.init_calibration()


def _first_difference(a, b):
  for i, (x, y) in enumerate(zip(a, b)):
    if x != y:
      return f'at {i}: ...{a[max(0, i - 80):i + 80]}... != ...{b[max(0, i - 80):i + 80]}...'
  return f'length {len(a)} != {len(b)}'


CASES = {
    # config_test.py:44-55
    'config_v4_custom': lambda: config.config_v4(
        fwd_bits=8, dlhs_bits=7, drhs_bits=6, rng_type='custom-1',
        dlhs_local_aqt=config.LocalAqt(contraction_axis_shard_count=2),
        drhs_local_aqt=config.LocalAqt(contraction_axis_shard_count=3),
        fwd_accumulator_dtype=utils.int16, dlhs_accumulator_dtype=utils.int8,
        drhs_accumulator_dtype=utils.int4),
    # config_test.py:470
    'config_v4_default': lambda: config.config_v4(),
    # config_test.py:646
    'config_fwd_fp8': lambda: config.config_fwd_fp8(),
}


@pytest.mark.parametrize('name', sorted(CASES))
def test_config_tree_prints_like_the_reference(name):
  cfg = CASES[name]()
  _init_all_calibrations(cfg)
  got = _normalise_actual(pprint.pformat(cfg))
  want = _normalise_golden(_golden(name))
  assert got == want, _first_difference(got, want)


def test_golden_files_are_the_three_trees():
  for name in CASES:
    text = _golden(name)
    assert text.startswith('DotGeneral(fwd=DotGeneralRaw(lhs=Tensor(') and 'apply_custom_vjp_on_jax=True)' in text

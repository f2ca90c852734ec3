"""Writes the configuration-tree goldens the reference's own test holds as data.

Reads aqt/jax/v2/config_test.py of the reference checkout AS TEXT (nothing is imported or run) and
copies out the three expected pprint strings (config_test.py:56-270, 275-469, 475-645): the
printed trees of config_v4(<custom arguments>), config_v4() and config_fwd_fp8() after
init_calibration() on all six quantizers.  Run once in a container that has the reference; the
.txt files next to this script are the fixtures tests/test_config_goldens.py compares against.

Usage: python tests/golden/make_config_goldens.py [/root/reference]
"""
import os
import re
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
NAMES = ['config_v4_custom', 'config_v4_default', 'config_fwd_fp8']


def main():
  ref = sys.argv[1] if len(sys.argv) > 1 else '/root/reference'
  text = open(os.path.join(ref, 'aqt/jax/v2/config_test.py')).read()
  found = re.findall(r'expected_cfg(?:_str)? = """(.*?)"""', text, flags=re.S)
  assert len(found) == len(NAMES), len(found)
  for name, s in zip(NAMES, found):
    with open(os.path.join(HERE, f'{name}.pprint.txt'), 'w') as f:
      f.write(s + '\n')
    print(name, len(s.splitlines()), 'lines')


if __name__ == '__main__':
  main()

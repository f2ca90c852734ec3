"""Builds libaqtx.so (the HIP kernels + C-ABI) for gfx950 with hipcc.

Usage: python -m aqt_amd.build [--jobs N]
The shared library lands in aqt_amd/lib/ next to the sources it was built from;
it is loaded with ctypes by aqt_amd._lib.
"""
import argparse
import concurrent.futures
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, 'csrc')
LIB_DIR = os.path.join(HERE, 'lib')
LIB_PATH = os.path.join(LIB_DIR, 'libaqtx.so')

SOURCES = ['capi.hip', 'quantize.hip', 'gemm_i8.hip', 'gemm_fp8.hip', 'decode_i8.hip', 'reduce.hip',
           'gemm_grouped.hip', 'fp_round.hip', 'im2col.hip']

HIPCC_FLAGS = [
    '--offload-arch=gfx950', '-O3', '-std=c++17', '-fPIC',
    # packed-FP32 VALU forms are kept out of generated code on purpose
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
    # every float product and sum of the reference rounds on its own: no fused multiply-add
    '-ffp-contract=off',
    '-Wno-unused-command-line-argument', '-Wno-pass-failed',
]


def _hipcc():
  exe = shutil.which('hipcc') or '/opt/rocm/bin/hipcc'
  if not os.path.exists(exe):
    raise RuntimeError('hipcc not found; a ROCm toolchain is required to build libaqtx.so')
  return exe


def _compile(src, obj):
  cmd = [_hipcc()] + HIPCC_FLAGS + ['-c', os.path.join(CSRC, src), '-o', obj]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError(f'hipcc failed on {src}:\n{res.stdout}\n{res.stderr}')
  return obj


def build_library(jobs=4, verbose=True):
  """Compiles every source and links aqt_amd/lib/libaqtx.so. Returns its path."""
  os.makedirs(LIB_DIR, exist_ok=True)
  obj_dir = os.path.join(LIB_DIR, 'obj')
  os.makedirs(obj_dir, exist_ok=True)
  sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
  objs = [os.path.join(obj_dir, s.replace('.hip', '.o')) for s in sources]
  with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
    list(pool.map(_compile, sources, objs))
  tmp = LIB_PATH + '.tmp'
  cmd = [_hipcc(), '--offload-arch=gfx950', '-shared', '-fPIC'] + objs + ['-o', tmp]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError(f'link failed:\n{res.stdout}\n{res.stderr}')
  os.replace(tmp, LIB_PATH)
  if verbose:
    print(f'built {LIB_PATH} from {len(sources)} sources', file=sys.stderr)
  return LIB_PATH


if __name__ == '__main__':
  ap = argparse.ArgumentParser()
  ap.add_argument('--jobs', type=int, default=4)
  build_library(ap.parse_args().jobs)

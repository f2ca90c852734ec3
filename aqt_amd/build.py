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

SOURCES = ['capi.hip', 'quantize.hip', 'gemm_i8.hip', 'gemm_mid.hip', 'gemm_fp8.hip', 'decode_i8.hip', 'decode_wo.hip', 'reduce.hip',
           'gemm_i8_frag.hip', 'gemm_wo.hip', 'gemm_grouped.hip', 'fp_round.hip', 'im2col.hip', 'scale_cast.hip']

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


FFI_SOURCE = 'aqtx_ffi.cc'
FFI_LIB_PATH = os.path.join(LIB_DIR, 'libaqtx_ffi.so')


def xla_ffi_include_dir():
  """Directory holding xla/ffi/api/ffi.h, or None.  The headers ship inside jaxlib
  (jax.ffi.include_dir()); AQTX_XLA_FFI_INCLUDE names another copy."""
  cands = []
  if os.environ.get('AQTX_XLA_FFI_INCLUDE'):
    cands.append(os.environ['AQTX_XLA_FFI_INCLUDE'])
  try:
    import jax.ffi  # pylint: disable=import-outside-toplevel
    cands.append(jax.ffi.include_dir())
  except Exception:  # jax is absent or too old to have jax.ffi
    pass
  for c in cands:
    if c and os.path.exists(os.path.join(c, 'xla', 'ffi', 'api', 'ffi.h')):
      return c
  return None


def build_ffi_shim(verbose=True):
  """Compiles the XLA FFI handlers (csrc/aqtx_ffi.cc) against libaqtx.so into
  aqt_amd/lib/libaqtx_ffi.so where the XLA FFI headers exist; returns its path, or None (with a
  message) where they do not.  Nothing stands in for missing headers."""
  inc = xla_ffi_include_dir()
  if inc is None:
    if verbose:
      print('XLA FFI headers (xla/ffi/api/ffi.h) not found: libaqtx_ffi.so not built '
            '(install jaxlib or set AQTX_XLA_FFI_INCLUDE)', file=sys.stderr)
    return None
  cmd = [_hipcc(), '-x', 'hip', '--offload-arch=gfx950', '-O2', '-std=c++17', '-fPIC', '-shared', '-I', inc,
         os.path.join(CSRC, FFI_SOURCE), '-L', LIB_DIR, '-laqtx', '-Wl,-rpath,$ORIGIN', '-o', FFI_LIB_PATH]
  res = subprocess.run(cmd, capture_output=True, text=True)
  if res.returncode != 0:
    raise RuntimeError(f'hipcc failed on {FFI_SOURCE}:\n{res.stdout}\n{res.stderr}')
  if verbose:
    print(f'built {FFI_LIB_PATH}', file=sys.stderr)
  return FFI_LIB_PATH


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
  try:
    build_ffi_shim(verbose)
  except RuntimeError as e:
    # the shim has never met a compiler where this library is developed (no XLA headers there): a failure to
    # build it must not take the library, which is complete without it, down with it
    print(f'warning: the XLA FFI shim did not build; libaqtx.so is unaffected\n{e}', file=sys.stderr)
  return LIB_PATH


if __name__ == '__main__':
  ap = argparse.ArgumentParser()
  ap.add_argument('--jobs', type=int, default=4)
  build_library(ap.parse_args().jobs)

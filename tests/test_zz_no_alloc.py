"""aqtx_decode_i8_static (the entry point that allocates nothing: its scratch is an array built into
the library's device code) against aqtx_decode_i8 on the same operands, through the C-ABI."""
import ctypes

import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from aqt_amd import ops

pytestmark = pytest.mark.gpu


def _operands(m, n, k, seed, dev, packed):
  g = torch.Generator(device='cpu').manual_seed(seed)
  x = (torch.randn(m, k, generator=g) * (1.0 + 20.0 * (torch.rand(m, k, generator=g) < 0.005))).to(torch.bfloat16).to(dev)
  if packed:
    w = torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.uint8).to(dev)
  else:
    w = torch.randint(-127, 128, (n, k), generator=g, dtype=torch.int8).to(dev)
  ws = (torch.rand(n, generator=g) * 1e-3 + 1e-5).to(dev)
  return x, w, ws


@pytest.mark.parametrize('packed', [False, True])
def test_static_scratch_matches_workspace_entry_point(gpu, packed):
  """Calls in a row on the built-in scratch, each smaller than the one before (so that it runs on whatever that
  one left behind), each bit for bit equal to aqtx_decode_i8.  plan.tuning asks for three K ranges per weight
  tile, so every call's workgroups meet through exchange words in the scratch, and those words overlap between
  the calls (they start at the same offset for every shape).  Every call leaves its exchange words zero, so what
  a later call finds there is zero whether or not its first kernel clears them; that the clearing copes with
  words that are NOT zero is shown on the same code with a workspace of random bytes
  (test_gpu_decode.py::test_decode_workspace_contract: the array's name cannot be written from a test)."""
  kw = dict(quant_bound=127.5, clip_bound=127.0, w_dtype=L.I4P if packed else L.I8, want_xq=True, tuning=3 | (2 << 8) | (1 << 16))
  for (m, n, k), seed in (((64, 4096, 4096), 1), ((24, 1000, 2048), 2), ((3, 256, 1024), 3)):
    x, w, ws = _operands(m, n, k, seed, gpu, packed)
    want = ops.decode(x, w, ws, **kw)
    got = ops.decode(x, w, ws, static_scratch=True, **kw)
    torch.cuda.synchronize()
    for a, b, name in zip(got, want, ('out', 'x_scale', 'xq')):
      assert torch.equal(a, b), (name, m, n, k)
    # once more: the scratch now holds this call's own leftovers
    again = ops.decode(x, w, ws, static_scratch=True, **kw)
    for a, b, name in zip(again, want, ('out', 'x_scale', 'xq')):
      assert torch.equal(a, b), (name, m, n, k, 'repeat')


def test_static_scratch_rejects_oversized_plans(gpu):
  plan = L.DecodePlan()
  plan.m, plan.n, plan.k = 8, 32768 + 16, 64
  plan.x_dtype = plan.x_scale_dtype = plan.out_dtype = L.BF16
  plan.w_scale_dtype = L.F32
  plan.quant_bound, plan.clip_bound, plan.w_dtype = 127.5, 127.0, L.I8
  rc = L.lib().aqtx_decode_i8_static(ctypes.byref(plan), None, None, None, None, None, None, None)
  assert rc != 0 and b'exceed the built-in scratch' in L.lib().aqtx_last_error()
  plan.n, plan.k = 64, 32768 + 64
  rc = L.lib().aqtx_decode_i8_static(ctypes.byref(plan), None, None, None, None, None, None, None)
  assert rc != 0 and b'exceed the built-in scratch' in L.lib().aqtx_last_error()


def test_static_scratch_makes_no_allocation(gpu):
  """torch's allocator sees nothing (it is not involved) and the driver's free-memory figure does
  not move across calls once the outputs exist."""
  x, w, ws = _operands(32, 2048, 4096, 5, gpu, False)
  plan = L.DecodePlan()
  plan.m, plan.n, plan.k = 32, 2048, 4096
  plan.x_dtype = plan.x_scale_dtype = plan.out_dtype = L.BF16
  plan.w_scale_dtype = L.F32
  plan.quant_bound, plan.clip_bound, plan.w_dtype = 127.5, 127.0, L.I8
  out = torch.empty((32, 2048), dtype=torch.bfloat16, device=gpu)
  xs = torch.empty(32, dtype=torch.float32, device=gpu)
  p = lambda t: ctypes.c_void_p(t.data_ptr())
  st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  call = lambda: L.check(L.lib().aqtx_decode_i8_static(ctypes.byref(plan), p(x), p(w), p(ws), None, p(xs), p(out), st))
  call()  # first call on the device: symbol lookup
  torch.cuda.synchronize()
  free0, _ = torch.cuda.mem_get_info()
  for _ in range(10):
    call()
  torch.cuda.synchronize()
  free1, _ = torch.cuda.mem_get_info()
  assert free1 == free0
  want, _ = ops.decode(x, w, ws, quant_bound=127.5, clip_bound=127.0)
  assert torch.equal(out, want)

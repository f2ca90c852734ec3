"""Tensor-level entry points over the aqtx C-ABI.

torch is used for device memory and the current HIP stream only; all arithmetic
happens in the HIP kernels.  Every function raises if a tensor is not on a GPU
or the library is missing -- there is no CPU path.
"""
from __future__ import annotations

import contextlib
import ctypes
import math
import os
from typing import Optional, Sequence

import numpy as np
import torch

from aqt_amd import _lib as L

_TORCH_TO_AQTX = {
    torch.float32: L.F32,
    torch.bfloat16: L.BF16,
    torch.int8: L.I8,
    torch.int32: L.I32,
}
_AQTX_TO_TORCH = {L.F32: torch.float32, L.BF16: torch.bfloat16, L.I32: torch.int32}


class KernelTimer:
  """Collects HIP-event pairs around chosen C-ABI launches on the launching stream.

  Used by the benchmark to time one kernel family inside a full step:
  `with KernelTimer('gemm') as t: ...; t.mean_ms()` after a synchronize.
  """
  active = None

  def __init__(self, family: str):
    self.family = family
    self.pairs = []

  def __enter__(self):
    KernelTimer.active = self
    return self

  def __exit__(self, *exc):
    KernelTimer.active = None
    return False

  def mean_ms(self):
    return sum(a.elapsed_time(b) for a, b in self.pairs) / max(len(self.pairs), 1)


class _timed:
  def __init__(self, family):
    t = KernelTimer.active
    self.t = t if (t is not None and t.family == family) else None

  def __enter__(self):
    if self.t is not None:
      self.a = torch.cuda.Event(enable_timing=True)
      self.a.record(torch.cuda.current_stream())

  def __exit__(self, *exc):
    if self.t is not None:
      b = torch.cuda.Event(enable_timing=True)
      b.record(torch.cuda.current_stream())
      self.t.pairs.append((self.a, b))
    return False


def aqtx_dtype(dt) -> int:
  if isinstance(dt, int):
    return dt
  try:
    return _TORCH_TO_AQTX[dt]
  except KeyError:
    raise TypeError(f'unsupported dtype for the aqtx kernels: {dt}') from None


def _ptr(t: Optional[torch.Tensor]):
  return None if t is None else ctypes.c_void_p(t.data_ptr())


def _stream():
  return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _require_gpu(*tensors):
  for t in tensors:
    if t is not None and not t.is_cuda:
      raise RuntimeError('aqt_amd kernels need tensors in GPU memory (got a CPU tensor); '
                         'there is no CPU fallback')


# One abs-max workspace per (device, stream), kept zeroed by the library between calls, so that
# the column and whole-tensor calibrations do not pay a clearing launch each time.
_QUANT_WS = {}


@contextlib.contextmanager
def private_workspaces(store: dict):
  """Calls made inside keep their abs-max workspaces in `store` instead of the process-wide table:
  a recorded HIP graph owns the workspace its kernels were recorded with."""
  global _QUANT_WS
  prev, _QUANT_WS = _QUANT_WS, store
  try:
    yield store
  finally:
    _QUANT_WS = prev


def _quantize_workspace(nbytes: int, device) -> torch.Tensor:
  key = (device.index, torch.cuda.current_stream(device).cuda_stream)
  ws = _QUANT_WS.get(key)
  if ws is None or ws.numel() < nbytes:
    ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
    _QUANT_WS[key] = ws
  return ws


def _decode_workspace(exchange_bytes: int, scratch_bytes: int, device) -> torch.Tensor:
  """The serving contraction's workspace for the current stream.  Its leading exchange words are
  zero between calls (the kernels reset what they use); the library keeps its other scratch in
  the last bytes, so the tensor holds the largest exchange size and the largest scratch size
  seen so far side by side."""
  key = ('decode', device.index, torch.cuda.current_stream(device).cuda_stream)
  ent = _QUANT_WS.get(key)
  if ent is None or ent[1] < exchange_bytes or ent[2] < scratch_bytes:
    ex = max(exchange_bytes, ent[1] if ent else 0, 1 << 20)
    sc = max(scratch_bytes, ent[2] if ent else 0, 1 << 20)
    ent = (torch.zeros(ex + sc, dtype=torch.uint8, device=device), ex, sc)
    _QUANT_WS[key] = ent
  return ent[0]


def quantize(
    x: torch.Tensor,
    *,
    reduce: int,
    out_dtype: int,
    quant_bound: float,
    clip_bound: float,
    compute_dtype=None,
    scale_dtype=None,
    group: int = 0,
    transpose_out: bool = False,
    noise: int = L.NOISE_NONE,
    key: Optional[Sequence[int]] = None,
    partitionable: bool = False,
    noise_strides: Optional[Sequence[int]] = None,
    noise_total: Optional[int] = None,
    prescale: Optional[torch.Tensor] = None,
    prescale_mode: int = L.PRESCALE_NONE,
    scale: Optional[torch.Tensor] = None,
    want_typed_scale: bool = False,
    key_device: Optional[torch.Tensor] = None,
    k_order: int = 0,
    want_other_axis_absmax: bool = False,
    absmax_partials: Optional[torch.Tensor] = None,
):
  """Calibrate (abs-max) and quantize a contiguous [batch, rows, cols] tensor.

  Returns (q, scale): q is int8 (or uint8 holding fp8 bytes), shaped
  [batch, rows, cols] or [batch, cols, rows] with transpose_out; scale is
  float32, shaped [batch, rows, cols/group] (REDUCE_COLS),
  [batch, rows/group, cols] (REDUCE_ROWS) or [batch] (REDUCE_ALL).
  `key_device` (a 2-word device tensor, or such a tensor passed as `key`) replaces `key`: the kernels read
  the key from device memory.
  `k_order` = L.K_EVEN_ODD8 stores every aligned group of 8 values along cols as elements
  0,2,4,6,1,3,5,7 (the lhs of gemm_grouped against a packed int4 rhs).
  With want_typed_scale a third element: the computed scales once more as a bf16 tensor of
  the same shape, written by the same kernels (None unless the scale dtype is bf16 and the
  scale is computed here).
  want_other_axis_absmax: where the plan allows it, the kernels also leave partial maxima of |q| along the axis
  that carries the scales (uint8 [parts, cols] for REDUCE_COLS, [parts, rows] for REDUCE_ROWS) in
  `q.other_axis_absmax`: what a later quantization of q over that axis takes as `absmax_partials` instead of
  reading q for its abs-max (the backward pass re-quantizes the forward residuals that way).
  """
  _require_gpu(x, prescale, scale)
  assert x.dim() == 3 and x.is_contiguous(), 'x must be a contiguous [batch, rows, cols] tensor'
  b, r, c = x.shape
  in_dt = aqtx_dtype(x.dtype)
  compute_dt = aqtx_dtype(compute_dtype) if compute_dtype is not None else in_dt
  scale_dt = aqtx_dtype(scale_dtype) if scale_dtype is not None else compute_dt
  plan = L.QuantPlan()
  plan.in_dtype, plan.compute_dtype, plan.scale_dtype, plan.out_dtype = in_dt, compute_dt, scale_dt, out_dtype
  plan.batch, plan.rows, plan.cols = b, r, c
  plan.reduce, plan.transpose_out, plan.group = reduce, int(transpose_out), group
  plan.quant_bound, plan.clip_bound = quant_bound, clip_bound
  plan.noise, plan.partitionable = noise, int(partitionable)
  if isinstance(key, torch.Tensor):  # a key held on the device (prng_split of a device key gives such keys)
    key_device, key = key, None
  if noise != L.NOISE_NONE:
    assert key is not None or key_device is not None, 'noise requested but no PRNG key given'
    if key_device is not None:  # uint32[2] (held as int32) in device memory, read by the kernels
      _require_gpu(key_device)
      assert key_device.numel() == 2 and key_device.element_size() == 4 and key_device.is_contiguous()
      plan.key_device = key_device.data_ptr()
    else:
      plan.key[0], plan.key[1] = int(key[0]), int(key[1])
    nsb, nsr, nsc = noise_strides if noise_strides is not None else (r * c, c, 1)
    plan.noise_stride_batch, plan.noise_stride_row, plan.noise_stride_col = nsb, nsr, nsc
    plan.noise_total = noise_total if noise_total is not None else b * r * c
  plan.prescale = prescale_mode
  if prescale is not None and prescale.dim() == 2 and prescale.shape[0] == b and b > 1:
    plan.prescale_stride_batch = prescale.shape[1]
  plan.scale_given = int(scale is not None)
  plan.out_k_order = k_order

  if reduce == L.REDUCE_COLS:
    sshape = (b, r, c // group if group else 1)
  elif reduce == L.REDUCE_ROWS:
    sshape = (b, r // group if group else 1, c)
  elif reduce == L.REDUCE_ALL:
    sshape = (b,)
  else:
    sshape = (1,)
  typed = None
  if scale is None:
    scale = torch.empty(sshape, dtype=torch.float32, device=x.device)
    if want_typed_scale and scale_dt == L.BF16:
      typed = torch.empty(sshape, dtype=torch.bfloat16, device=x.device)
      plan.scale_typed = typed.data_ptr()
  else:
    assert scale.dtype == torch.float32 and scale.is_contiguous() and tuple(scale.shape) == sshape
  fp8 = out_dtype in (L.E4M3, L.E5M2)
  qshape = (b, c, r) if transpose_out else (b, r, c)
  q = torch.empty(qshape, dtype=torch.uint8 if fp8 else torch.int8, device=x.device)
  if prescale is not None:
    assert prescale.dtype == torch.float32 and prescale.is_contiguous()
  lib = L.lib()
  other = None
  if want_other_axis_absmax:
    parts = int(lib.aqtx_quantize_other_axis_parts(ctypes.byref(plan)))
    if parts > 0:
      other = torch.empty((parts, c if reduce == L.REDUCE_COLS else r), dtype=torch.uint8, device=x.device)
      plan.other_axis_absmax = other.data_ptr()
  if absmax_partials is not None:
    _require_gpu(absmax_partials)
    assert (absmax_partials.dtype == torch.uint8 and absmax_partials.is_contiguous() and absmax_partials.dim() == 2
            and absmax_partials.shape[1] == c and not plan.scale_given), (absmax_partials.shape, x.shape)
    plan.absmax_partials, plan.absmax_parts = absmax_partials.data_ptr(), absmax_partials.shape[0]
  ws_bytes = lib.aqtx_quantize_workspace_bytes(ctypes.byref(plan))
  ws = _quantize_workspace(ws_bytes, x.device) if ws_bytes else None
  plan.workspace_zeroed = int(ws is not None)
  try:
    L.check(lib.aqtx_quantize(ctypes.byref(plan), _ptr(x), _ptr(prescale), _ptr(q), _ptr(scale),
                              _ptr(ws), ws.numel() if ws is not None else 0, _stream()))
  except Exception:
    _QUANT_WS.clear()  # a failed launch sequence may have left abs-max words behind
    raise
  if other is not None:
    q.other_axis_absmax = other
  return (q, scale, typed) if want_typed_scale else (q, scale)


# aqtx_gemm_plan.tuning of every gemm() call: 0 = the library's choice; 4 | 8 = waves per workgroup
# of the int8 kernel on 256 x 256 tiles, 128 = the kernel on 128 x 128 tiles (the parity tests run all three).
GEMM_TUNING = 0

# aqtx_gemm_plan.accumulate of fp8 gemm() calls that do not say: L.ACC_FAST = the fp8 matrix instruction (products
# of every 8 consecutive k aligned to the largest of them and cut off 2^-13 below it), L.ACC_F32 = both operands
# widened to bf16 on their way to the matrix cores, sums within the error bound of a float32 summation at half the
# rate.  AQTX_FP8_ACCUMULATE=f32 in the environment selects the latter for a whole process.
FP8_ACCUMULATE = L.ACC_F32 if os.environ.get('AQTX_FP8_ACCUMULATE', '').lower() == 'f32' else L.ACC_FAST


def gemm(
    a: torch.Tensor,
    b: torch.Tensor,
    *,
    row_scale: Optional[torch.Tensor],
    col_scale: Optional[torch.Tensor],
    out_dtype,
    dequant_dtype=None,
    scale_dtype=None,
    row_scale_dtype=None,
    col_scale_dtype=None,
    scale_order: int = L.SCALE_ROW_THEN_COL,
    a_dtype: int = L.I8,
    b_dtype: int = L.I8,
    want_acc: bool = False,
    group_offsets: Optional[torch.Tensor] = None,
    a_k_order: int = 0,
    k_split: int = 0,
    b_layout: int = L.W_ROWS,
    accumulate: Optional[int] = None,
):
  """C[b] = dequant(A[b] @ B[b]^T) for A [batch, m, k], B [batch, n, k] (k contiguous).

  accumulate (fp8 operands only; None = FP8_ACCUMULATE): L.ACC_FAST contracts with the fp8 matrix
  instruction, L.ACC_F32 through bf16 with float32-like sums at half the rate.

  b_layout = L.W_FRAGMENTS (int8 operands, batch 1): B is the flat buffer tile_weight made of one weight
  [n, k] (or of its packed int4 form), the copy the serving kernels stream; n is then col_scale's length.

  k_split (int8 operands; results do not depend on it): 0 = the library decides whether slices of k go
  to workgroups of their own (few output tiles, long k), 1 = never, S > 1 = S slices.

  b_dtype = L.I4P: B is uint8 [batch, n, k/2], int4 values packed two per byte (pack_i4); with
  a_k_order = L.K_EVEN_ODD8 A was written by quantize(k_order=L.K_EVEN_ODD8).

  With `group_offsets` (int32 device tensor [groups + 1], ascending): a ragged product.  A is
  [1, m, k], B [groups, n, k]; group g multiplies rows off[g]:off[g+1] of A with B[g] into the
  same rows of C [1, m, n], in one launch; rows outside every group are left as allocated
  (zero-initialised here).

  int8 operands use the int32 MFMA path, fp8 operands (uint8 tensors holding
  e4m3fn/e5m2 bytes) the float32 one.  `scale_dtype` names the dtype of both scale
  vectors; row_scale_dtype / col_scale_dtype override it per side.  Returns C, or
  (C, acc) with want_acc.
  """
  _require_gpu(a, b, row_scale, col_scale)
  batch, m, k = a.shape
  if b_layout == L.W_FRAGMENTS:
    assert batch == 1 and group_offsets is None and col_scale is not None and b.is_contiguous() and a.stride(2) == 1
    n = col_scale.shape[-1]
    assert b.numel() * b.element_size() == L.lib().aqtx_tile_weight_bytes(n, k, b_dtype), (b.shape, n, k)
    b_batches, ldb, stride_b = 1, 0, 0
  else:
    assert a.dim() == 3 and b.dim() == 3 and a.shape[2] == (2 * b.shape[2] if b_dtype == L.I4P else b.shape[2])
    assert a.shape[0] == b.shape[0] or group_offsets is not None
    assert a.stride(2) == 1 and b.stride(2) == 1, 'the contraction axis must be contiguous'
    n = b.shape[1]
    b_batches, ldb, stride_b = b.shape[0], b.stride(1), b.stride(0)
  if group_offsets is not None:
    assert a.shape[0] == 1 and group_offsets.dtype == torch.int32 and group_offsets.is_cuda
    assert group_offsets.numel() == b.shape[0] + 1 and group_offsets.is_contiguous()
  fp8 = a_dtype in (L.E4M3, L.E5M2)
  out_dt = aqtx_dtype(out_dtype)
  dq_dt = aqtx_dtype(dequant_dtype) if dequant_dtype is not None else (out_dt if out_dt != L.I32 else L.F32)
  sc_dt = aqtx_dtype(scale_dtype) if scale_dtype is not None else dq_dt
  alloc = torch.zeros if group_offsets is not None else torch.empty
  c = alloc((batch, m, n), dtype=_AQTX_TO_TORCH[out_dt], device=a.device)
  acc = None
  if want_acc:
    acc = torch.empty((batch, m, n), dtype=torch.float32 if fp8 else torch.int32, device=a.device)
  plan = L.GemmPlan()
  plan.batch, plan.m, plan.n, plan.k = (b_batches if group_offsets is not None else batch), m, n, k
  plan.group_offsets = group_offsets.data_ptr() if group_offsets is not None else None
  plan.lda, plan.ldb, plan.ldc = a.stride(1), ldb, n
  plan.stride_a, plan.stride_b, plan.stride_c = a.stride(0), stride_b, m * n
  plan.b_layout = b_layout
  plan.a_dtype, plan.b_dtype = a_dtype, b_dtype
  plan.out_dtype, plan.dequant_dtype = out_dt, dq_dt
  plan.row_scale_dtype = aqtx_dtype(row_scale_dtype) if row_scale_dtype is not None else sc_dt
  plan.col_scale_dtype = aqtx_dtype(col_scale_dtype) if col_scale_dtype is not None else sc_dt
  plan.scale_order = scale_order
  plan.tuning = GEMM_TUNING
  plan.a_k_order = a_k_order
  plan.k_split = 1 if fp8 else k_split
  plan.accumulate = (FP8_ACCUMULATE if accumulate is None else accumulate) if fp8 else L.ACC_FAST
  for s, shape in ((row_scale, (batch, m)), (col_scale, (b_batches, n))):
    if s is not None:
      assert s.dtype == torch.float32 and s.is_contiguous() and tuple(s.shape) == shape, (tuple(s.shape), shape)
  plan.row_scale_stride_b, plan.col_scale_stride_b = m, n
  fn = L.lib().aqtx_gemm_fp8 if fp8 else L.lib().aqtx_gemm_i8
  slabs = None
  if not fp8:
    slices = L.lib().aqtx_gemm_i8_k_slices(ctypes.byref(plan))
    if slices > 1:  # slices of k leave their partial sums in slabs of a scratch array
      slabs = torch.empty((slices, batch, m, n), dtype=torch.int32, device=a.device)
      plan.k_split_workspace, plan.k_split_workspace_bytes = slabs.data_ptr(), slabs.numel() * 4
  with _timed('gemm'):
    L.check(fn(ctypes.byref(plan), _ptr(a), _ptr(b), _ptr(row_scale), _ptr(col_scale), _ptr(c),
               _ptr(acc), _stream()))
  return (c, acc) if want_acc else c


def ragged_offsets(group_sizes, m: int, device) -> torch.Tensor:
  """[0, s0, s0+s1, ...] as int32 on the device, clamped to the m rows there are; computed on the
  device when the sizes live there (no host round trip)."""
  sizes = group_sizes if isinstance(group_sizes, torch.Tensor) else torch.tensor(list(group_sizes), dtype=torch.int32)
  sizes = sizes.to(device=device, dtype=torch.int32)
  offs = torch.zeros(sizes.numel() + 1, dtype=torch.int32, device=device)
  offs[1:] = torch.cumsum(sizes, 0)
  return torch.clamp(offs, max=m)


def gemm_weight_only(a: torch.Tensor, b: torch.Tensor, col_scale: torch.Tensor, *, col_scale_dtype=torch.float32,
                     b_dtype: int = L.I8, b_layout: int = L.W_ROWS, tuning: Optional[int] = None):
  """Weight-only contraction C[b] = bf16(bf16(A[b] @ float(B[b])^T) * col_scale[b]) for bf16 A [batch, m, k] that
  stays unquantized and int8 B [batch, n, k] (k contiguous in both), any m; `col_scale` is float32 [batch, n]
  holding values of `col_scale_dtype`.  float32 sums; the weight is never copied as bf16.  tuning (None =
  GEMM_TUNING): 128 = 128 x 128 tiles, 8 = 256 x 256 tiles, 16 = those walked by one workgroup per CU; every
  choice sums k in the same order, so the results do not depend on it."""
  _require_gpu(a, b, col_scale)
  assert a.dim() == 3 and a.dtype == torch.bfloat16 and a.stride(2) == 1
  batch, m, k = a.shape
  if b_layout == L.W_FRAGMENTS:  # the flat buffer tile_weight made of one int8 weight [n, k]
    n = col_scale.shape[-1]
    assert batch == 1 and b.is_contiguous() and b.numel() * b.element_size() == L.lib().aqtx_tile_weight_bytes(n, k, L.I8)
    ldb = stride_b = 0
  else:
    assert b.dim() == 3 and a.shape[2] == b.shape[2] and a.shape[0] == b.shape[0] and b.dtype == torch.int8 and b.stride(2) == 1
    n, ldb, stride_b = b.shape[1], b.stride(1), b.stride(0)
  assert col_scale.dtype == torch.float32 and col_scale.is_contiguous() and tuple(col_scale.shape) == (batch, n)
  c = torch.empty((batch, m, n), dtype=torch.bfloat16, device=a.device)
  plan = L.GemmPlan()
  plan.batch, plan.m, plan.n, plan.k = batch, m, n, k
  plan.lda, plan.ldb, plan.ldc = a.stride(1), ldb, n
  plan.stride_a, plan.stride_b, plan.stride_c = a.stride(0), stride_b, m * n
  plan.b_layout = b_layout
  plan.a_dtype, plan.b_dtype = L.BF16, b_dtype
  plan.out_dtype = plan.dequant_dtype = plan.row_scale_dtype = L.BF16
  plan.col_scale_dtype = aqtx_dtype(col_scale_dtype)
  plan.col_scale_stride_b = n
  plan.tuning = GEMM_TUNING if tuning is None else tuning
  if plan.tuning == 4:
    plan.tuning = 8  # the weight-only kernel has one workgroup shape on the large tiles
  with _timed('gemm'):
    L.check(L.lib().aqtx_gemm_weight_only(ctypes.byref(plan), _ptr(a), _ptr(b), _ptr(col_scale), _ptr(c), _stream()))
  return c


def decode_weight_only(x: torch.Tensor, w_q: torch.Tensor, w_scale: torch.Tensor, *, w_scale_dtype=torch.float32,
                       w_dtype: int = L.I8, w_layout: int = L.W_ROWS, out_dtype=None, tuning: int = 0):
  """Weight-only serving contraction out = dequant(x @ float(w_q)^T) for bf16 x [m <= 64, k] that stays
  unquantized and w_q int8 [n, k] (or packed int4 uint8 [n, k/2], or either re-laid by tile_weight);
  `w_scale` is float32 [n] holding values of `w_scale_dtype`.  float32 sums."""
  _require_gpu(x, w_q, w_scale)
  packed = w_dtype == L.I4P
  assert x.dim() == 2 and x.is_contiguous() and w_q.is_contiguous() and x.dtype == torch.bfloat16
  m, k = x.shape
  if w_layout == L.W_FRAGMENTS:
    n = w_scale.numel()
    assert w_q.numel() * w_q.element_size() == L.lib().aqtx_tile_weight_bytes(n, k, w_dtype), (w_q.shape, n, k)
  else:
    assert w_q.dim() == 2 and k == w_q.shape[1] * (2 if packed else 1), (x.shape, w_q.shape)
    n = w_q.shape[0]
  assert w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == n
  out_dtype = out_dtype if out_dtype is not None else x.dtype
  plan = L.DecodePlan()
  plan.m, plan.n, plan.k = m, n, k
  plan.x_dtype = aqtx_dtype(x.dtype)
  plan.x_scale_dtype = plan.x_dtype
  plan.w_scale_dtype = aqtx_dtype(w_scale_dtype)
  plan.out_dtype = aqtx_dtype(out_dtype)
  plan.quant_bound = plan.clip_bound = 1.0
  plan.w_dtype, plan.w_layout, plan.tuning = w_dtype, w_layout, tuning
  out = torch.empty((m, n), dtype=out_dtype, device=x.device)
  need = L.lib().aqtx_decode_weight_only_workspace_bytes(ctypes.byref(plan))
  ws = torch.empty(need, dtype=torch.uint8, device=x.device) if need else None
  with _timed('decode'):
    L.check(L.lib().aqtx_decode_weight_only(ctypes.byref(plan), _ptr(x), _ptr(w_q), _ptr(w_scale), _ptr(out),
                                            _ptr(ws) if ws is not None else None, need, _stream()))
  return out


def decode(x: torch.Tensor, w_q: torch.Tensor, w_scale: torch.Tensor, *, quant_bound: float,
           clip_bound: float, x_scale_dtype=None, w_scale_dtype=torch.float32, want_xq: bool = False,
           w_dtype: int = L.I8, tuning: int = 0, static_scratch: bool = False, w_layout: int = L.W_ROWS):
  """Serving contraction out = dequant(quant(x) @ w_q^T) for x [m <= 64, k], w_q int8 [n, k], or
  uint8 [n, k/2] holding packed int4 (w_dtype=I4P, the pack_i4 layout).

  The activations get per-token dynamic int8 quantisation; `w_scale` is float32 [n] holding
  values of `w_scale_dtype`.  Returns (out [m, n] of x.dtype, x_scale float32 [m]) and, with
  want_xq, the quantized activations as a third element.  With static_scratch the call goes
  through aqtx_decode_i8_static: the library's built-in device scratch instead of a workspace
  tensor (n, k <= 32768; calls on one GPU must not overlap).
  """
  _require_gpu(x, w_q, w_scale)
  packed = w_dtype == L.I4P
  assert x.dim() == 2 and x.is_contiguous() and w_q.is_contiguous()
  m, k = x.shape
  if w_layout == L.W_FRAGMENTS:  # the output of tile_weight: a flat buffer; n is the number of scales
    n = w_scale.numel()
    assert w_q.numel() * w_q.element_size() == L.lib().aqtx_tile_weight_bytes(n, k, w_dtype), (w_q.shape, n, k)
  else:
    assert w_q.dim() == 2 and k == w_q.shape[1] * (2 if packed else 1), (x.shape, w_q.shape)
    assert w_q.dtype == (torch.uint8 if packed else torch.int8)
    n = w_q.shape[0]
  assert w_scale.dtype == torch.float32 and w_scale.is_contiguous() and w_scale.numel() == n
  plan = L.DecodePlan()
  plan.m, plan.n, plan.k = m, n, k
  plan.x_dtype = aqtx_dtype(x.dtype)
  plan.x_scale_dtype = aqtx_dtype(x_scale_dtype if x_scale_dtype is not None else x.dtype)
  plan.w_scale_dtype = aqtx_dtype(w_scale_dtype)
  plan.out_dtype = plan.x_dtype
  plan.quant_bound, plan.clip_bound = float(quant_bound), float(clip_bound)
  plan.w_dtype = w_dtype
  plan.tuning = tuning  # launch-shape override for measurements; results do not depend on it
  plan.w_layout = w_layout
  if static_scratch:
    out = torch.empty((m, n), dtype=x.dtype, device=x.device)
    x_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
    xq = torch.empty((m, k), dtype=torch.int8, device=x.device) if want_xq else None
    with _timed('decode'):
      L.check(L.lib().aqtx_decode_i8_static(ctypes.byref(plan), _ptr(x), _ptr(w_q), _ptr(w_scale), _ptr(xq),
                                            _ptr(x_scale), _ptr(out), _stream()))
    return (out, x_scale, xq) if want_xq else (out, x_scale)
  ws_bytes = int(L.lib().aqtx_decode_workspace_bytes(ctypes.byref(plan)))
  ex_bytes = int(L.lib().aqtx_decode_exchange_bytes(ctypes.byref(plan)))
  # one workspace per (device, stream), zero before its first use and left zero by every call
  ws = _decode_workspace(ex_bytes, ws_bytes - ex_bytes, x.device)
  plan.workspace_zeroed = 1
  out = torch.empty((m, n), dtype=x.dtype, device=x.device)
  x_scale = torch.empty((m,), dtype=torch.float32, device=x.device)
  xq = torch.empty((m, k), dtype=torch.int8, device=x.device) if want_xq else None
  try:
    with _timed('decode'):
      L.check(L.lib().aqtx_decode_i8(ctypes.byref(plan), _ptr(x), _ptr(w_q), _ptr(w_scale), _ptr(xq),
                                     _ptr(x_scale), _ptr(out), _ptr(ws), ws.numel(), _stream()))
  except Exception:
    _QUANT_WS.clear()  # a failed launch sequence may have left partial sums behind
    raise
  return (out, x_scale, xq) if want_xq else (out, x_scale)


def decode_check(device=None) -> None:
  """Raises if a serving call on this stream's workspace gave up waiting for its quantized activations (which
  leaves that call's outputs unwritten).  Synchronizes the stream: for the points where a caller synchronizes
  anyway; the workspace is dropped after an error, so the next call starts from a clean one."""
  device = torch.device('cuda', torch.cuda.current_device()) if device is None else torch.device(device)
  ent = _QUANT_WS.get(('decode', device.index, torch.cuda.current_stream(device).cuda_stream))
  if ent is None:
    return
  try:
    L.check(L.lib().aqtx_decode_i8_check(_ptr(ent[0]), ent[0].numel(), _stream()))
  except Exception:
    _QUANT_WS.clear()
    raise


def tile_weight(w_q: torch.Tensor, w_dtype: int = L.I8) -> torch.Tensor:
  """A frozen weight [n, k] (int8, or packed int4 uint8 [n, k/2]) in MFMA fragment order: the layout
  decode(..., w_layout=W_FRAGMENTS) streams fastest.  Returns a flat uint8 buffer."""
  _require_gpu(w_q)
  packed = w_dtype == L.I4P
  assert w_q.dim() == 2 and w_q.is_contiguous() and w_q.dtype == (torch.uint8 if packed else torch.int8)
  n, k = w_q.shape[0], w_q.shape[1] * (2 if packed else 1)
  out = torch.empty(int(L.lib().aqtx_tile_weight_bytes(n, k, w_dtype)), dtype=torch.uint8, device=w_q.device)
  L.check(L.lib().aqtx_tile_weight(_ptr(w_q), _ptr(out), n, k, w_dtype, _stream()))
  return out


def read_probe(buf: torch.Tensor, out: Optional[torch.Tensor] = None, *, workgroups: int = 512, loads_in_flight: int = 4,
               cache_policy: int = 2, stamps: Optional[torch.Tensor] = None) -> torch.Tensor:
  """Streams `buf` once through the library's read-only kernel (a measurement aid, not part of any product
  path); returns the checksum words, one per workgroup.  workgroups = 0: one workgroup per chunk of
  256 * loads_in_flight * 16 bytes; otherwise that many workgroups walk the chunks round-robin.  `stamps`
  (int64 [2 * workgroups]) receives every workgroup's first and last device-clock reading (read_probe_span_us)."""
  _require_gpu(buf)
  assert buf.is_contiguous()
  nbytes = buf.numel() * buf.element_size()
  if out is None:
    out = torch.zeros(65536, dtype=torch.int32, device=buf.device)
  assert out.numel() >= 65536 and (stamps is None or (stamps.dtype == torch.int64 and stamps.numel() >= 2 * 65536))
  L.check(L.lib().aqtx_read_probe(_ptr(buf), nbytes, workgroups, loads_in_flight, cache_policy, _ptr(out), _ptr(stamps),
                                  None, _stream()))
  return out


def read_probe_workgroups(nbytes: int, workgroups: int, loads_in_flight: int) -> int:
  """Workgroups a read_probe launch has (it never has more than chunks)."""
  nchunks = -(-nbytes // (256 * loads_in_flight * 16))
  return nchunks if workgroups == 0 else min(workgroups, nchunks)


def read_probe_span_us(stamps: torch.Tensor, workgroups: int) -> float:
  """Span of the read_probe launch that wrote `stamps`: last workgroup's end minus first workgroup's start."""
  khz = ctypes.c_int32(0)
  L.check(L.lib().aqtx_read_probe(None, 0, 0, 4, 0, None, None, ctypes.byref(khz), None))
  s = stamps[:2 * workgroups].cpu().numpy().reshape(-1, 2)
  return float(int(s[:, 1].max()) - int(s[:, 0].min())) * 1e3 / khz.value


def pack_i4(q: torch.Tensor) -> torch.Tensor:
  """int4 values held one per int8 byte, last axis even -> uint8 tensor with the last axis halved."""
  _require_gpu(q)
  assert q.dtype == torch.int8 and q.is_contiguous() and q.shape[-1] % 2 == 0
  out = torch.empty(q.shape[:-1] + (q.shape[-1] // 2,), dtype=torch.uint8, device=q.device)
  L.check(L.lib().aqtx_pack_i4(_ptr(q), _ptr(out), q.numel(), _stream()))
  return out


def gemm_grouped(a: torch.Tensor, b: torch.Tensor, *, row_scale: torch.Tensor, col_scale: torch.Tensor,
                 group: int, out_dtype, row_scale_dtype=None, col_scale_dtype=None, a_dtype: int = L.I8,
                 b_dtype: int = L.I8, a_k_order: int = 0, row_scale_by_row: bool = False, tuning: int = 0):
  """C = cast(sum_g dequant_g(A_g @ B_g^T)) for A int8 [m, k], B int8 [n, k] (or packed int4
  uint8 [n, k/2] with b_dtype=I4P), row_scale float32 [k/group, m] ([m, k/group] with
  row_scale_by_row), col_scale float32 [k/group, n].  a_k_order = L.K_EVEN_ODD8: A was written by
  quantize(k_order=L.K_EVEN_ODD8) (packed rhs only)."""
  _require_gpu(a, b, row_scale, col_scale)
  m, k = a.shape
  n = b.shape[0]
  packed = b_dtype == L.I4P
  assert a.stride(1) == 1 and b.stride(1) == 1 and b.shape[1] == (k // 2 if packed else k)
  groups = k // group
  for s_, shape in ((row_scale, (m, groups) if row_scale_by_row else (groups, m)), (col_scale, (groups, n))):
    assert s_.dtype == torch.float32 and s_.is_contiguous() and tuple(s_.shape) == shape, tuple(s_.shape)
  out_dt = aqtx_dtype(out_dtype)
  plan = L.GroupedGemmPlan()
  plan.m, plan.n, plan.k, plan.group = m, n, k, group
  plan.lda, plan.ldb, plan.ldc = a.stride(0), b.stride(0), n
  plan.a_dtype, plan.b_dtype, plan.out_dtype = a_dtype, b_dtype, out_dt
  plan.row_scale_dtype = aqtx_dtype(row_scale_dtype) if row_scale_dtype is not None else out_dt
  plan.col_scale_dtype = aqtx_dtype(col_scale_dtype) if col_scale_dtype is not None else out_dt
  plan.a_k_order, plan.row_scale_by_row = a_k_order, int(row_scale_by_row)
  plan.tuning = tuning  # kernel override for tests and measurements; results do not depend on it
  c = torch.empty((m, n), dtype=_AQTX_TO_TORCH[out_dt], device=a.device)
  with _timed('gemm_grouped'):
    L.check(L.lib().aqtx_gemm_i8_grouped(ctypes.byref(plan), _ptr(a), _ptr(b), _ptr(row_scale),
                                         _ptr(col_scale), _ptr(c), _stream()))
  return c


def sum_tiles(x: torch.Tensor) -> torch.Tensor:
  """Sum over the leading axis of a contiguous bf16/f32 tensor: float32 accumulation in index
  order, one rounding (jnp.sum semantics for the per-tile outputs of a tiled dot_general)."""
  _require_gpu(x)
  assert x.is_contiguous() and x.dim() >= 1
  tiles = x.shape[0]
  out = torch.empty(x.shape[1:], dtype=x.dtype, device=x.device)
  L.check(L.lib().aqtx_sum_tiles(_ptr(x), _ptr(out), tiles, out.numel(), aqtx_dtype(x.dtype), _stream()))
  return out


def _window_plan(x: torch.Tensor, kernel, strides, pads, dilation):
  """aqtx_im2col_plan of the windows of x [n, *spatial, c]; returns (plan, output spatial sizes)."""
  rank = x.dim() - 2
  plan = L.Im2colPlan()
  plan.n, plan.c, plan.rank = x.shape[0], x.shape[-1], rank
  out_sizes = []
  for d in range(rank):
    eff = (int(kernel[d]) - 1) * int(dilation[d]) + 1
    span = int(pads[d][0]) + x.shape[1 + d] + int(pads[d][1]) - eff
    o = span // int(strides[d]) + 1 if span >= 0 else 0
    out_sizes.append(o)
    plan.in_size[d], plan.kernel[d], plan.stride[d] = x.shape[1 + d], int(kernel[d]), int(strides[d])
    plan.dilation[d], plan.pad_lo[d], plan.out_size[d] = int(dilation[d]), int(pads[d][0]), o
  return plan, out_sizes


def im2col_i8(x: torch.Tensor, kernel, strides, pads, dilation):
  """Windows of an int8 tensor [n, *spatial, c] as a matrix [n * positions, taps * c] (zeros in the
  padding); returns (matrix, output spatial sizes).  `pads` are (low, high) pairs."""
  _require_gpu(x)
  assert x.dtype == torch.int8 and x.is_contiguous() and 3 <= x.dim() <= 5
  rank = x.dim() - 2
  plan, out_sizes = _window_plan(x, kernel, strides, pads, dilation)
  rows = x.shape[0] * math.prod(out_sizes)
  k = math.prod(int(t) for t in kernel[:rank]) * x.shape[-1]
  out = torch.empty((rows, k), dtype=torch.int8, device=x.device)
  L.check(L.lib().aqtx_im2col_i8(ctypes.byref(plan), _ptr(x), _ptr(out), _stream()))
  return out, out_sizes


def conv_i8_supported(x: torch.Tensor) -> bool:
  """Whether conv_i8 takes this input: features a multiple of 128, less than 2 GiB."""
  return x.shape[-1] > 0 and x.shape[-1] % 128 == 0 and x.numel() < 2 ** 31


def conv_i8(x: torch.Tensor, w: torch.Tensor, kernel, strides, pads, dilation, *, row_scale, col_scale, out_dtype,
            row_scale_dtype=None, col_scale_dtype=None, scale_order: int = L.SCALE_ROW_THEN_COL):
  """dequant(windows(x) @ w^T) in one launch, the windows read in place: x int8 [n, *spatial, c], w int8
  [features_out, taps * c] (tap order row-major, features innermost), row_scale float32 [n * positions],
  col_scale float32 [features_out].  Same bits as im2col_i8 + gemm.  Returns ([n * positions, features_out],
  output spatial sizes)."""
  _require_gpu(x, w, row_scale, col_scale)
  assert x.dtype == torch.int8 and w.dtype == torch.int8 and x.is_contiguous() and 3 <= x.dim() <= 5
  assert w.dim() == 2 and w.stride(1) == 1 and conv_i8_supported(x)
  rank = x.dim() - 2
  win, out_sizes = _window_plan(x, kernel, strides, pads, dilation)
  m = x.shape[0] * math.prod(out_sizes)
  k = math.prod(int(t) for t in kernel[:rank]) * x.shape[-1]
  n = w.shape[0]
  assert w.shape[1] == k
  out_dt = aqtx_dtype(out_dtype)
  plan = L.GemmPlan()
  plan.batch, plan.m, plan.n, plan.k = 1, m, n, k
  plan.lda, plan.ldb, plan.ldc = k, w.stride(0), n
  plan.a_dtype = plan.b_dtype = L.I8
  plan.out_dtype = plan.dequant_dtype = out_dt
  plan.row_scale_dtype = aqtx_dtype(row_scale_dtype) if row_scale_dtype is not None else out_dt
  plan.col_scale_dtype = aqtx_dtype(col_scale_dtype) if col_scale_dtype is not None else out_dt
  plan.scale_order = scale_order
  plan.k_split = 1
  for s_, shape in ((row_scale, (m,)), (col_scale, (n,))):
    if s_ is not None:
      assert s_.dtype == torch.float32 and s_.is_contiguous() and tuple(s_.shape) == shape, (tuple(s_.shape), shape)
  c = torch.empty((m, n), dtype=_AQTX_TO_TORCH[out_dt], device=x.device)
  L.check(L.lib().aqtx_conv_i8(ctypes.byref(win), ctypes.byref(plan), _ptr(x), _ptr(w), _ptr(row_scale),
                               _ptr(col_scale), _ptr(c), _stream()))
  return c, out_sizes


def fp_round(x: torch.Tensor, *, nexp: int, nmant: int, has_subnormals: bool, key=None,
             stochastic_rounding: bool = False, noise_mod: Optional[int] = None,
             partitionable: bool = False, radix: int = 2) -> torch.Tensor:
  """x (bf16 or f32, any shape) rounded to an emulated small float in the same dtype
  (radix = 4: to the powers of 4 from 4^-3 to 4^3, bf16 only; nexp / nmant are then not read).

  Stochastic rounding draws jax.random.bits(key, x.shape, uint16); `noise_mod` replaces the draw
  by the index along the last axis (which must have that extent).
  """
  _require_gpu(x)
  x = x.contiguous()
  out = torch.empty_like(x)
  plan = L.FpRoundPlan()
  plan.count = x.numel()
  plan.dtype = aqtx_dtype(x.dtype)
  plan.nexp, plan.nmant, plan.has_subnormals = int(nexp), int(nmant), int(bool(has_subnormals))
  plan.partitionable = int(partitionable)
  plan.radix = int(radix)
  k = None
  if not stochastic_rounding:
    plan.mode = L.FP_NEAREST
  elif noise_mod is not None:
    assert x.dim() >= 1 and x.shape[-1] == noise_mod
    plan.mode, plan.noise_mod = L.FP_NOISE_INDEX, int(noise_mod)
  else:
    assert key is not None, 'stochastic rounding requested but the key is None'
    key = _host_key(key, 'fp_round')
    plan.mode = L.FP_NOISE_JAX_BITS
    k = (ctypes.c_uint32 * 2)(int(key[0]), int(key[1]))
  L.check(L.lib().aqtx_fp_round(ctypes.byref(plan), _ptr(x), _ptr(out), k, _stream()))
  return out


def prng_split(key, num: int, partitionable: bool = False):
  """jax.random.split(key, num) on raw uint32[2] key data: on the host for a numpy key (returns numpy
  [num, 2]); for a key that is a 2-word device tensor, by a kernel, into a device tensor [num, 2] (no host
  round trip: the split can be recorded into a HIP graph and follows the key's value on every replay)."""
  if isinstance(key, torch.Tensor):
    _require_gpu(key)
    assert key.numel() == 2 and key.element_size() == 4 and key.is_contiguous()
    out = torch.empty((num, 2), dtype=key.dtype, device=key.device)
    L.check(L.lib().aqtx_prng_split(_ptr(key), num, int(partitionable), _ptr(out), _stream()))
    return out
  k = (ctypes.c_uint32 * 2)(int(key[0]), int(key[1]))
  out = (ctypes.c_uint32 * (2 * num))()
  L.check(L.lib().aqtx_prng_split_host(k, num, int(partitionable), out))
  return np.frombuffer(out, dtype=np.uint32).reshape(num, 2).copy()


def _host_key(key, who: str):
  if isinstance(key, torch.Tensor):
    raise TypeError(f'{who}: a PRNG key held on the device is only read by the fused quantize kernels; pass a host key')
  return key


def random_bits(key, n: int, bit_width: int = 32, partitionable: bool = False, device='cuda'):
  """jax.random.bits(key, (n,), uint{bit_width}) generated on the GPU."""
  key = _host_key(key, 'random_bits')
  k = (ctypes.c_uint32 * 2)(int(key[0]), int(key[1]))
  out = torch.empty(n, dtype=torch.int16 if bit_width == 16 else torch.int32, device=device)
  _require_gpu(out)
  L.check(L.lib().aqtx_random_bits(k, n, bit_width, int(partitionable), _ptr(out), _stream()))
  return out


def scale_cast(x: torch.Tensor, factors=(), *, out_dtype, in_dtype=None, finish_clip=None,
               finish_round: int = 0) -> torch.Tensor:
  """out = cast(x) times up to two factors, each with one value per (batch, row) or per (batch, column).

  x is [batch, rows, cols], contiguous: int8 / fp8 bytes (`in_dtype` says which: I8, I4, E4M3, E5M2; default
  from x.dtype) or bf16 / f32.  `factors`: tuples (vector, axis, dtype, recast[, reciprocal]) with vector float32
  [batch, rows] / [batch, cols] (or [rows] / [cols], shared between the batch entries), axis L.FACTOR_ROWS |
  L.FACTOR_COLS, dtype the dtype its values are held in, recast whether the running value is cast to out_dtype
  first, reciprocal whether the factor divides (QTensor.quant).  finish_clip / finish_round (1: half to even,
  2: floor + 0.5): the clipping and rounding of integer numerics on the result, which stays a float.
  """
  _require_gpu(x)
  assert x.dim() == 3 and x.is_contiguous() and len(factors) <= 2
  b, r, c = x.shape
  plan = L.ScalePlan()
  if in_dtype is None:
    in_dtype = L.I8 if x.dtype in (torch.int8, torch.uint8) else aqtx_dtype(x.dtype)
  plan.in_dtype, plan.out_dtype = in_dtype, aqtx_dtype(out_dtype)
  plan.batch, plan.rows, plan.cols = b, r, c
  plan.factors = len(factors)
  ptrs = [None, None]
  plan.finish_clip = float(finish_clip) if finish_clip else 0.0
  plan.finish_round = finish_round
  for i, (vec, axis, dt, recast, *more) in enumerate(factors):
    plan.factor_reciprocal[i] = int(bool(more and more[0]))
    n = r if axis == L.FACTOR_ROWS else c
    assert vec.dtype == torch.float32 and vec.is_contiguous() and vec.numel() in (n, b * n), (vec.shape, axis, x.shape)
    _require_gpu(vec)
    plan.factor_axis[i], plan.factor_dtype[i], plan.factor_recast[i] = axis, aqtx_dtype(dt), int(bool(recast))
    plan.factor_stride_b[i] = n if vec.numel() == b * n and b > 1 else 0
    ptrs[i] = _ptr(vec)
  out = torch.empty((b, r, c), dtype=_AQTX_TO_TORCH[plan.out_dtype], device=x.device)
  L.check(L.lib().aqtx_scale_cast(ctypes.byref(plan), _ptr(x), ptrs[0], ptrs[1], _ptr(out), _stream()))
  return out


def dequantize(q: torch.Tensor, scale: torch.Tensor, *, reduce: int, q_dtype: int, out_dtype,
               scale_dtype=None, group: int = 0, transposed: bool = False):
  """out = cast(q) * scale for q as written by `quantize` (one scale).

  q is [batch, rows, cols] (or [batch, cols, rows] when transposed); the result is
  [batch, rows, cols] of out_dtype.
  """
  _require_gpu(q, scale)
  assert q.dim() == 3 and q.is_contiguous() and scale.dtype == torch.float32 and scale.is_contiguous()
  b, r, c = (q.shape[0], q.shape[2], q.shape[1]) if transposed else q.shape
  out_dt = aqtx_dtype(out_dtype)
  plan = L.QuantPlan()
  plan.in_dtype = plan.compute_dtype = out_dt
  plan.scale_dtype = aqtx_dtype(scale_dtype) if scale_dtype is not None else out_dt
  plan.out_dtype = q_dtype
  plan.batch, plan.rows, plan.cols = b, r, c
  plan.reduce, plan.transpose_out, plan.group = reduce, int(transposed), group
  plan.quant_bound = plan.clip_bound = 1.0
  out = torch.empty((b, r, c), dtype=_AQTX_TO_TORCH[out_dt], device=q.device)
  L.check(L.lib().aqtx_dequantize(ctypes.byref(plan), _ptr(q), _ptr(scale), _ptr(out), _stream()))
  return out

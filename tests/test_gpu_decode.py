"""GPU parity: aqtx_decode_i8 (serving with a frozen int8 weight) against the oracle."""
import numpy as np
import pytest
import torch

from aqt_amd import ops
from oracle import aqt_ref as R
from oracle import numerics as nm
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _oracle_decode(x, dt, wq, w_scale, w_sdt):
  """quant(x) per token, int32 contraction, QTensor.dequant with [x scale, w scale]."""
  q = R.QuantizerCfg(bits=8)
  xqt = R.quantize(x, dt, q, calibration_axes=[1])
  acc = (xqt.qvalue.astype(np.int64) @ wq.astype(np.int64).T).astype(np.int32)
  xs = xqt.scale[0].reshape(-1, 1)
  out = R.dequant(R.QTensor(acc, 'i32', [xs, w_scale.reshape(1, -1)], None, dt,
                            scale_dtypes=[xqt.scale_dtype, w_sdt]))
  return out, xqt.qvalue.astype(np.int8), xqt.scale[0].reshape(-1)


def _weights(n, k, seed, w_sdt):
  rng = np.random.default_rng(seed)
  wq = rng.integers(-127, 128, size=(n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(2e-4) + np.float32(1e-5), w_sdt)
  return wq, ws


# aqtx_decode_plan.tuning bits 16-19: the library's choice of kernels; the many-token kernel for every m, its first
# workgroups quantizing the tokens; the same with the quantisation in a launch of its own
PATHS = pytest.mark.parametrize('path', [0, 1 << 16, 2 << 16], ids=['auto', 'producers', 'two_launches'])


@PATHS
@pytest.mark.parametrize('m', [1, 2, 3, 8, 16, 17, 32, 40, 64])
@pytest.mark.parametrize('n,k', [(256, 1024), (200, 464), (4096, 4096), (24, 8192 + 4096)])
@pytest.mark.parametrize('dt,w_sdt', [('bf16', 'f32'), ('bf16', 'bf16'), ('f32', 'f32')])
def test_decode_matches_oracle(gpu, m, n, k, dt, w_sdt, path):
  if (n, k) == (4096, 4096) and (dt, w_sdt) != ('bf16', 'f32'):
    pytest.skip('large shape once')
  x = U.rand((m, k), dt, 100 + m, outliers=True)
  wq, ws = _weights(n, k, 7, w_sdt)
  want, xq_want, xs_want = _oracle_decode(x, dt, wq, ws, w_sdt)
  out, xs, xq = ops.decode(U.to_dev(x, dt, gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                           quant_bound=127.5, clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt], want_xq=True, tuning=path)
  np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
  np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  ops.decode_check()


def test_decode_wait_that_expires_is_reported_and_nothing_hangs(gpu):
  """Error path of the launch whose first workgroups quantize the tokens, forced from the host: the workgroups
  that contract are told to wait for one token more than there are, for a microsecond.  Every kernel ends
  normally, decode_check reports the expired wait, and the next call (on a fresh workspace) is right again."""
  m, n, k = 8, 512, 1024
  x = U.rand((m, k), 'bf16', 77)
  wq, ws = _weights(n, k, 8, 'f32')
  args = (U.to_dev(x, 'bf16', gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu))
  ops.decode(*args, quant_bound=127.5, clip_bound=127.0, tuning=(1 << 16) | (1 << 20))
  with pytest.raises(RuntimeError, match='expired'):
    ops.decode_check()
  ops.decode_check()  # the mark is gone with the workspace
  want, _, _ = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  out, _ = ops.decode(*args, quant_bound=127.5, clip_bound=127.0, tuning=1 << 16)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  ops.decode_check()


@pytest.mark.parametrize('m', [20, 64])
def test_decode_wide_weight(gpu, m):
  """n >= 12288 takes the 64-rows-per-workgroup shape; k is not a multiple of the 256-byte chunk."""
  n, k = 12352 + 24, 336
  x = U.rand((m, k), 'bf16', 5)
  wq, ws = _weights(n, k, 9, 'f32')
  want, _, _ = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  out, _ = ops.decode(U.to_dev(x, 'bf16', gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                      quant_bound=127.5, clip_bound=127.0)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)


def test_decode_equals_quantize_plus_gemm(gpu):
  """Same result as the training-shape kernels on the same operands."""
  from aqt_amd import _lib as L
  m, n, k = 64, 512, 4096
  x = U.to_dev(U.rand((m, k), 'bf16', 3), 'bf16', gpu)
  wq, ws = _weights(n, k, 4, 'bf16')
  wq_t, ws_t = torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu)
  out, xs = ops.decode(x, wq_t, ws_t, quant_bound=127.5, clip_bound=127.0, w_scale_dtype=torch.bfloat16)
  xq, xs2 = ops.quantize(x[None], reduce=L.REDUCE_COLS, out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)
  ref = ops.gemm(xq, wq_t[None], row_scale=xs2.reshape(1, m), col_scale=ws_t.reshape(1, n),
                 out_dtype=torch.bfloat16, scale_dtype=torch.bfloat16)
  assert torch.equal(xs, xs2.reshape(-1))
  assert torch.equal(out, ref[0])


def test_decode_rejects_bad_plans(gpu):
  x = torch.zeros((65, 64), dtype=torch.bfloat16, device=gpu)
  w = torch.zeros((16, 64), dtype=torch.int8, device=gpu)
  s = torch.ones(16, device=gpu)
  with pytest.raises(Exception, match='exceeds 64'):
    ops.decode(x, w, s, quant_bound=127.5, clip_bound=127.0)
  with pytest.raises(Exception, match='multiple of 16'):
    ops.decode(x[:4, :24].contiguous(), w[:, :24].contiguous(), s, quant_bound=127.5, clip_bound=127.0)


@PATHS
@pytest.mark.parametrize('m', [1, 2, 8, 16, 17, 32, 33, 64])
@pytest.mark.parametrize('n,k', [(256, 1024), (200, 480), (40, 32), (4096, 4096), (72, 8192)])
@pytest.mark.parametrize('dt,w_sdt', [('bf16', 'f32'), ('bf16', 'bf16'), ('f32', 'f32')])
def test_decode_packed_int4_matches_oracle(gpu, m, n, k, dt, w_sdt, path):
  """int4 weights packed two per byte (aqtx_pack_i4 layout): same numbers as the int8-held
  form, half the weight bytes."""
  from aqt_amd import _lib as L
  if (n, k) == (4096, 4096) and (dt, w_sdt) != ('bf16', 'f32'):
    pytest.skip('large shape once')
  x = U.rand((m, k), dt, 200 + m, outliers=True)
  rng = np.random.default_rng(11)
  wq = rng.integers(-7, 8, size=(n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(3e-3) + np.float32(1e-4), w_sdt)
  want, xq_want, xs_want = _oracle_decode(x, dt, wq, ws, w_sdt)
  wq_t = torch.from_numpy(wq).to(gpu)
  packed = ops.pack_i4(wq_t)
  assert packed.shape == (n, k // 2) and packed.dtype == torch.uint8
  out, xs, xq = ops.decode(U.to_dev(x, dt, gpu), packed, torch.from_numpy(ws).to(gpu), quant_bound=127.5,
                           clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt], want_xq=True, w_dtype=L.I4P, tuning=path)
  np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
  np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  # and the int8-held int4 weight through the int8 kernels gives the same
  if k % 16 == 0:
    out8, _ = ops.decode(U.to_dev(x, dt, gpu), wq_t, torch.from_numpy(ws).to(gpu), quant_bound=127.5,
                         clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt], w_dtype=L.I4)
    assert torch.equal(out, out8)


@pytest.mark.parametrize('m', [20, 64])
def test_decode_packed_int4_wide_weight(gpu, m):
  """n >= 8192: each wave takes two 16-row weight blocks; n is not a multiple of 32."""
  from aqt_amd import _lib as L
  n, k = 8192 + 40, 160
  x = U.rand((m, k), 'bf16', 6)
  rng = np.random.default_rng(12)
  wq = rng.integers(-7, 8, size=(n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(3e-3) + np.float32(1e-4), 'f32')
  want, _, _ = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  out, _ = ops.decode(U.to_dev(x, 'bf16', gpu), ops.pack_i4(torch.from_numpy(wq).to(gpu)),
                      torch.from_numpy(ws).to(gpu), quant_bound=127.5, clip_bound=127.0, w_dtype=L.I4P)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)


@pytest.mark.parametrize('m', [1, 2])
@pytest.mark.parametrize('k', [4112, 8192, 8208])
@pytest.mark.parametrize('dt,w_sdt', [('bf16', 'f32'), ('f32', 'f32'), ('bf16', 'bf16')])
def test_decode_one_or_two_rows_long_k(gpu, m, k, dt, w_sdt):
  """One or two tokens take the kernel that quantizes the activations itself; above k = 4096
  each thread holds two pieces per row, above 8192 the two-kernel path runs.  The quantized
  activations and scales it writes out are the oracle's."""
  n = 72
  x = U.rand((m, k), dt, 300 + m, outliers=True)
  wq, ws = _weights(n, k, 8, w_sdt)
  want, xq_want, xs_want = _oracle_decode(x, dt, wq, ws, w_sdt)
  out, xs, xq = ops.decode(U.to_dev(x, dt, gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                           quant_bound=127.5, clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt], want_xq=True)
  np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
  np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  out2, _ = ops.decode(U.to_dev(x, dt, gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                       quant_bound=127.5, clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt])
  assert torch.equal(out, out2)


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('m,n,k', [(5, 200, 464 + 16), (24, 1000, 2048), (64, 520, 4096), (40, 4096, 1024)])
def test_decode_every_launch_shape_gives_the_same_bits(gpu, packed, m, n, k):
  """plan.tuning only chooses the launch shape (rows per weight tile, K ranges per tile that meet
  through the int32 atomic exchange, K steps in flight): every choice must return the oracle's
  bits, and so must the one- and two-token kernel's arithmetic when m <= 2 is sent down the
  two-kernel path."""
  from aqt_amd import _lib as L
  if packed:
    k = (k + 31) // 32 * 32
  x = U.rand((m, k), 'bf16', 400 + m, outliers=True)
  rng = np.random.default_rng(13)
  lim = 7 if packed else 127
  wq = rng.integers(-lim, lim + 1, size=(n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(2e-4) + np.float32(1e-5), 'f32')
  want, xq_want, xs_want = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  w_t = torch.from_numpy(wq).to(gpu)
  if packed:
    w_t = ops.pack_i4(w_t)
  for splits in (1, 2, 3, 7):
    for nb in (1, 2, 4):
      for depth in (2, 4, 15):
        tuning = splits | (nb << 8) | (depth << 12)
        out, xs, xq = ops.decode(U.to_dev(x, 'bf16', gpu), w_t, torch.from_numpy(ws).to(gpu), quant_bound=127.5,
                                 clip_bound=127.0, want_xq=True, w_dtype=L.I4P if packed else L.I8, tuning=tuning)
        np.testing.assert_array_equal(out.float().cpu().numpy(), want, err_msg=hex(tuning))
        np.testing.assert_array_equal(xq.cpu().numpy(), xq_want, err_msg=hex(tuning))
        np.testing.assert_array_equal(xs.cpu().numpy(), xs_want, err_msg=hex(tuning))


@pytest.mark.parametrize('m', [3, 4])
@pytest.mark.parametrize('k', [480, 4096, 4112, 8192])
@pytest.mark.parametrize('dt,w_sdt', [('bf16', 'f32'), ('f32', 'f32'), ('bf16', 'bf16')])
def test_decode_three_or_four_rows_one_kernel(gpu, m, k, dt, w_sdt):
  """Three or four tokens against a weight of at most 256 row blocks take the 16-wave kernel that
  quantizes the activations itself (two pieces per thread above k = 4096); forcing the two-kernel
  path gives the same bits, and both give the oracle's outputs, scales and quantized activations."""
  n = 200
  x = U.rand((m, k), dt, 700 + m, outliers=True)
  wq, ws = _weights(n, k, 9, w_sdt)
  want, xq_want, xs_want = _oracle_decode(x, dt, wq, ws, w_sdt)
  for tuning in (0, 1 << 16):
    out, xs, xq = ops.decode(U.to_dev(x, dt, gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                             quant_bound=127.5, clip_bound=127.0, w_scale_dtype=U.TORCH_DT[w_sdt], want_xq=True,
                             tuning=tuning)
    np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
    np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)
    np.testing.assert_array_equal(out.float().cpu().numpy(), want)


@pytest.mark.parametrize('m', [1, 2])
def test_decode_two_kernel_path_for_one_or_two_tokens(gpu, m):
  n, k = 328, 2048
  x = U.rand((m, k), 'bf16', 500 + m, outliers=True)
  wq, ws = _weights(n, k, 14, 'f32')
  want, xq_want, xs_want = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  out, xs, xq = ops.decode(U.to_dev(x, 'bf16', gpu), torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu),
                           quant_bound=127.5, clip_bound=127.0, want_xq=True, tuning=1 << 16)
  np.testing.assert_array_equal(out.float().cpu().numpy(), want)
  np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
  np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)


def test_decode_workspace_contract(gpu):
  """A caller-owned workspace with arbitrary contents (workspace_zeroed = 0) and one kept zeroed
  across calls of different shapes (workspace_zeroed = 1) give the same bits; the exchange words
  are zero again after every call."""
  import ctypes
  from aqt_amd import _lib as L
  shapes = [(64, 4096, 512), (8, 136, 8192), (33, 1000, 1024), (64, 264, 4096)]
  plans = []
  for m, n, k in shapes:
    p = L.DecodePlan()
    p.m, p.n, p.k = m, n, k
    p.x_dtype = p.x_scale_dtype = p.out_dtype = L.BF16
    p.w_scale_dtype = L.F32
    p.quant_bound, p.clip_bound, p.w_dtype = 127.5, 127.0, L.I8
    # three K ranges per tile: the exchange is in use for every shape; the many-token kernel for every m, so that the
    # calls on the kept workspace have their first workgroups quantize the tokens (control words in use as well)
    p.tuning = 3 | (2 << 8) | (1 << 16)
    plans.append(p)
  lib = L.lib()
  ex = max(int(lib.aqtx_decode_exchange_bytes(ctypes.byref(p))) for p in plans)
  rest = max(int(lib.aqtx_decode_workspace_bytes(ctypes.byref(p))) - int(lib.aqtx_decode_exchange_bytes(ctypes.byref(p)))
             for p in plans)
  kept = torch.zeros(ex + rest, dtype=torch.uint8, device=gpu)
  ptr = lambda t: ctypes.c_void_p(t.data_ptr())
  st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
  for p, (m, n, k) in zip(plans, shapes):
    x = U.to_dev(U.rand((m, k), 'bf16', 600 + m), 'bf16', gpu)
    wq, ws = _weights(n, k, 15, 'f32')
    w_t, ws_t = torch.from_numpy(wq).to(gpu), torch.from_numpy(ws).to(gpu)
    outs = []
    for zeroed in (0, 1):
      p.workspace_zeroed = zeroed
      if zeroed:
        wsp = kept
      else:
        wsp = torch.randint(0, 256, (int(lib.aqtx_decode_workspace_bytes(ctypes.byref(p))),), dtype=torch.uint8, device=gpu)
      out = torch.empty((m, n), dtype=torch.bfloat16, device=gpu)
      xs = torch.empty(m, dtype=torch.float32, device=gpu)
      L.check(lib.aqtx_decode_i8(ctypes.byref(p), ptr(x), ptr(w_t), ptr(ws_t), None, ptr(xs), ptr(out), ptr(wsp),
                                 wsp.numel(), st))
      outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[0], outs[1]), (m, n, k)
    assert int(kept[:ex].max()) == 0, 'exchange words were left non-zero'
    want, _, _ = _oracle_decode(U.rand((m, k), 'bf16', 600 + m), 'bf16', wq, ws, 'f32')
    np.testing.assert_array_equal(outs[1].float().cpu().numpy(), want)


def _fragment_order(w_bytes):
  """numpy statement of the fragment layout: [16-row block][64-byte step][lane = c*16 + r][16 bytes]
  with lane (r, c) holding bytes [64*step + 16*c, +16) of row 16*block + r, zeros outside."""
  n, kb = w_bytes.shape
  nb, ns = (n + 15) // 16, (kb + 63) // 64
  padded = np.zeros((nb * 16, ns * 64), dtype=np.uint8)
  padded[:n, :kb] = w_bytes
  t = padded.reshape(nb, 16, ns, 4, 16)        # block, r, step, c, byte
  return np.ascontiguousarray(t.transpose(0, 2, 3, 1, 4)).reshape(-1)  # block, step, c, r, byte


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('n,k', [(16, 64), (200, 480), (4096, 1024), (72, 8192 + 32)])
def test_tile_weight_layout(gpu, packed, n, k):
  from aqt_amd import _lib as L
  rng = np.random.default_rng(21)
  w = rng.integers(0, 256, size=(n, k // 2 if packed else k)).astype(np.uint8)
  src = torch.from_numpy(w).to(gpu)
  got = ops.tile_weight(src if packed else src.view(torch.int8), L.I4P if packed else L.I8)
  np.testing.assert_array_equal(got.cpu().numpy(), _fragment_order(w))


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('m', [1, 2, 3, 16, 33, 64])
@pytest.mark.parametrize('n,k', [(256, 1024), (200, 480), (4096, 4096), (72, 8192)])
def test_decode_fragment_ordered_weight(gpu, packed, m, n, k):
  """The weight in fragment order (aqtx_tile_weight) gives the oracle's bits on every path: the
  one/two-token kernel, 16/32/64-row tiles, K ranges meeting through the exchange."""
  from aqt_amd import _lib as L
  if packed:
    k = (k + 31) // 32 * 32
  x = U.rand((m, k), 'bf16', 700 + m, outliers=True)
  rng = np.random.default_rng(22)
  lim = 7 if packed else 127
  wq = rng.integers(-lim, lim + 1, size=(n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(2e-4) + np.float32(1e-5), 'f32')
  want, xq_want, xs_want = _oracle_decode(x, 'bf16', wq, ws, 'f32')
  w_t = torch.from_numpy(wq).to(gpu)
  wd = L.I8
  if packed:
    w_t, wd = ops.pack_i4(w_t), L.I4P
  tiled = ops.tile_weight(w_t, wd)
  for tuning in (0, 2 | (4 << 8), 3 | (1 << 8) | (4 << 12)):
    out, xs, xq = ops.decode(U.to_dev(x, 'bf16', gpu), tiled, torch.from_numpy(ws).to(gpu), quant_bound=127.5,
                             clip_bound=127.0, want_xq=True, w_dtype=wd, w_layout=L.W_FRAGMENTS, tuning=tuning)
    np.testing.assert_array_equal(out.float().cpu().numpy(), want, err_msg=hex(tuning))
    np.testing.assert_array_equal(xq.cpu().numpy(), xq_want)
    np.testing.assert_array_equal(xs.cpu().numpy(), xs_want)


@pytest.mark.parametrize('workgroups,loads,policy', [(0, 16, 2), (0, 2, 0), (3, 4, 2), (512, 8, 3), (7, 16, 1)])
def test_read_probe_reads_every_byte(gpu, workgroups, loads, policy):
  """The read-only kernel's checksum words: workgroup w holds the XOR of all 32-bit words of the chunks
  w, w + workgroups, ... (chunks of 256 * loads * 16 bytes; the last one ragged)."""
  buf = torch.randint(-2 ** 31, 2 ** 31 - 1, (11 * 16384 + 52,), dtype=torch.int32, device=gpu)
  stamps = torch.zeros(2 * 65536, dtype=torch.int64, device=gpu)
  got = ops.read_probe(buf, workgroups=workgroups, loads_in_flight=loads, cache_policy=policy, stamps=stamps)
  words = buf.cpu().numpy().view(np.uint32)
  cw = 256 * loads * 4
  chunks = [np.bitwise_xor.reduce(words[i:i + cw]) for i in range(0, len(words), cw)]
  nwg = ops.read_probe_workgroups(buf.numel() * 4, workgroups, loads)
  want = [np.bitwise_xor.reduce(np.asarray(chunks[w::nwg], dtype=np.uint32)) for w in range(nwg)]
  np.testing.assert_array_equal(got.cpu().numpy().view(np.uint32)[:nwg], np.asarray(want, dtype=np.uint32))
  assert not got[nwg:].any()
  assert 0.0 < ops.read_probe_span_us(stamps, nwg) < 1e4


# ---- weight-only serving (the lhs stays bf16; float32 sums: tolerance, not bits) ----------------------------
@pytest.mark.gpu
@pytest.mark.parametrize('tuning', [0, 3 << 4, (8 << 4) | 1])  # the library's choice; 3 slices of k; 8 slices, 16-row tiles
@pytest.mark.parametrize('layout', ['rows', 'fragments'])
@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('w_sdt', ['bf16', 'f32'])
@pytest.mark.parametrize('m,n,k', [(1, 200, 4096), (5, 16, 64), (16, 1024, 528 + 16 * 31), (17, 72, 2048), (33, 4096, 1024),
                                   (64, 300, 4096)])
def test_weight_only_decode_within_float_summation_error(gpu, m, n, k, w_sdt, packed, layout, tuning):
  """out = bf16(bf16(sum_k x w) * scale) with the sum in float32 in the kernel's own order.  Tolerance, stated:
  against the sum taken exactly (float64; every product of a bf16 and an int8 is exact), a float32 sum in any
  order is off by less than d = k * 2^-24 * sum_k |x w|.  Every later step (the two roundings, the product with
  a positive scale) is monotone, so each output must lie between the same steps applied to exact - d and to
  exact + d; where the terms cancel that is many ulps of a small result, elsewhere less than one.  99 % of the
  outputs must equal the steps applied to the exact sum.  With slices of k (forced through `tuning`, or chosen
  for the last two shapes) the partial sums are added in slice order: the same bound."""
  from aqt_amd import _lib as L
  if packed and k % 32 != 0:
    pytest.skip('packed int4 needs k % 32 == 0')
  rng = np.random.default_rng(41)
  x = nm.to_bf16(rng.standard_normal((m, k), dtype=np.float32))
  lo, hi = (-8, 8) if packed else (-127, 128)
  w = rng.integers(lo, hi, (n, k)).astype(np.int8)
  ws = nm.cast(np.abs(rng.standard_normal(n).astype(np.float32)) * np.float32(2e-3) + np.float32(1e-4), w_sdt)
  exact = x.astype(np.float64) @ w.astype(np.float64).T
  slack = k * 2.0 ** -24 * (np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T)

  def later_steps(total):
    prod = nm.to_bf16(total.astype(np.float32)).astype(np.float64) * ws.astype(np.float64)[None, :]
    prod = nm.cast(prod.astype(np.float32), w_sdt)
    return nm.to_bf16(prod).astype(np.float64)

  want, low, high = later_steps(exact), later_steps(exact - slack), later_steps(exact + slack)
  wt = torch.from_numpy(w).to(gpu)
  w_dtype = L.I8
  if packed:
    wt, w_dtype = ops.pack_i4(wt), L.I4P
  w_layout = L.W_ROWS
  if layout == 'fragments':
    wt, w_layout = ops.tile_weight(wt, w_dtype), L.W_FRAGMENTS
  got = ops.decode_weight_only(torch.from_numpy(x).to(torch.bfloat16).to(gpu), wt, torch.from_numpy(ws.astype(np.float32)).to(gpu),
                               w_scale_dtype=U.TORCH_DT[w_sdt], w_dtype=w_dtype, w_layout=w_layout, tuning=tuning)
  got = got.float().cpu().numpy().astype(np.float64)
  assert ((low <= got) & (got <= high)).all(), np.argwhere((got < low) | (got > high))[:8]
  assert (got == want).mean() >= 0.99


@pytest.mark.gpu
def test_weight_only_serving_takes_the_kernel(gpu, monkeypatch):
  """A float lhs of at most 64 rows against a frozen int8 rhs goes to the streaming weight-only kernel; more rows
  take the tiled weight-only kernel, or, with WEIGHT_ONLY_FLOAT_COPY on, the float product on the promoted
  weight.  Same numbers to float summation order."""
  from aqt_amd.v2 import aqt_dot_general as aqt, config
  dt = 'bf16'
  MATMUL = (((1,), (0,)), ((), ()))
  cfg = config.set_context(aqt.dot_general_make(None, 8), None, None)
  w = U.to_dev(U.rand((1024, 520), dt, 3, 0.05), dt, gpu)
  x_small, x_large = U.to_dev(U.rand((24, 1024), dt, 1), dt, gpu), U.to_dev(U.rand((80, 1024), dt, 2), dt, gpu)
  calls = []
  for name in ('decode_weight_only', 'gemm_weight_only'):
    real = getattr(ops, name)
    monkeypatch.setattr(ops, name, lambda *a, _real=real, _name=name, **k: (calls.append(_name), _real(*a, **k))[1])
  with torch.no_grad():
    monkeypatch.setattr(aqt, 'WEIGHT_ONLY_FLOAT_COPY', True)
    _, (_, wq) = cfg.dg_core(x_small, w, None, None, MATMUL)
    out_small, (lqt, _) = cfg.dg_core(x_small, torch.zeros_like(w), None, wq, MATMUL)
    out_large, _ = cfg.dg_core(x_large, torch.zeros_like(w), None, wq, MATMUL)
    assert calls == ['decode_weight_only'] and lqt.qvalue is x_small and lqt.scale == []
    monkeypatch.setattr(aqt, 'WEIGHT_ONLY_FLOAT_COPY', False)
    out_large_kernel, _ = cfg.dg_core(x_large, torch.zeros_like(w), None, wq, MATMUL)
    assert calls == ['decode_weight_only', 'gemm_weight_only']
  wf = wq.qvalue.float() * wq.scale[0].float()
  for out, x in ((out_small, x_small), (out_large, x_large), (out_large_kernel, x_large)):
    want = (x.float() @ wf).cpu().numpy()
    np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=2.0 ** -6, atol=2.0 ** -6 * np.abs(want).max())
  assert (out_large_kernel != out_large).float().mean() < 0.02  # both round a float32 sum to bf16


@pytest.mark.gpu
def test_weight_only_serving_many_tokens_narrow_weight(gpu):
  """48 tokens against a frozen int8 weight of 512 rows and k = 8192: the layer call goes to the weight-only kernel
  with k in slices (a workspace is asked for and lent), and agrees with the float product on the dequantized
  weight to float32 summation order."""
  from aqt_amd import _lib as L
  from aqt_amd.v2 import aqt_dot_general as aqt, config
  import ctypes
  dt = 'bf16'
  MATMUL = (((1,), (0,)), ((), ()))
  plan = L.DecodePlan()
  plan.m, plan.n, plan.k = 48, 512, 8192
  plan.x_dtype = plan.x_scale_dtype = plan.out_dtype = plan.w_scale_dtype = L.BF16
  plan.quant_bound = plan.clip_bound = 1.0
  plan.w_dtype, plan.w_layout = L.I8, L.W_FRAGMENTS
  assert L.lib().aqtx_decode_weight_only_workspace_bytes(ctypes.byref(plan)) == 8 * 48 * 512 * 4
  cfg = config.set_context(aqt.dot_general_make(None, 8), None, None)
  w = U.to_dev(U.rand((8192, 512), dt, 3, 0.05), dt, gpu)
  x = U.to_dev(U.rand((48, 8192), dt, 1), dt, gpu)
  with torch.no_grad():
    _, (_, wq) = cfg.dg_core(x, w, None, None, MATMUL)
    out, _ = cfg.dg_core(x, torch.zeros_like(w), None, wq, MATMUL)
  want = (x.float() @ (wq.qvalue.float() * wq.scale[0].float())).cpu().numpy()
  np.testing.assert_allclose(out.float().cpu().numpy(), want, rtol=2.0 ** -6, atol=2.0 ** -6 * np.abs(want).max())

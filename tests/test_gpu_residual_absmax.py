"""The partial maxima a forward quantizer leaves for the backward pass's re-quantization of its values over the
other axis (_maybe_use_fwd_quant, aqt_dot_general.py:675-729): what they hold, that a quantization which takes them
gives the bits of one that reads the tensor for its abs-max, and that a training step uses them."""
import numpy as np
import pytest
import torch

from aqt_amd import _lib as L
from aqt_amd import ops
from aqt_amd.v2 import aqt_dot_general as aqt
from aqt_amd.v2 import config
from aqt_amd.v2 import utils
from tests import gpu_util as U

pytestmark = pytest.mark.gpu

KW = dict(out_dtype=L.I8, quant_bound=127.5, clip_bound=127.0)
MATMUL = (((1,), (0,)), ((), ()))


def _x(shape, dt, seed, gpu):
  return U.to_dev(U.rand(shape, dt, seed, outliers=True), dt, gpu)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('rows,cols', [(300, 1024), (2500, 4096), (64, 8192), (1100, 520)])
def test_row_quantizer_leaves_column_maxima(gpu, dt, rows, cols):
  x = _x((1, rows, cols), dt, 1, gpu)
  q0, s0 = ops.quantize(x, reduce=L.REDUCE_COLS, **KW)
  q1, s1 = ops.quantize(x, reduce=L.REDUCE_COLS, want_other_axis_absmax=True, **KW)
  assert torch.equal(q0, q1) and torch.equal(s0, s1)
  parts = q1.other_axis_absmax
  assert parts.dtype == torch.uint8 and parts.shape == (min(rows, 1792), cols)
  qa = np.abs(q1[0].cpu().numpy().astype(np.int32))
  P = parts.shape[0]
  for p in (0, 1, P // 2, P - 1):
    np.testing.assert_array_equal(parts[p].cpu().numpy(), qa[p::P].max(axis=0))
  np.testing.assert_array_equal(parts.cpu().numpy().max(axis=0), qa.max(axis=0))


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
@pytest.mark.parametrize('rows,cols', [(128, 64), (512, 320), (4096, 1792)])
def test_tile_quantizer_leaves_row_maxima(gpu, dt, rows, cols):
  """One scale per column, q written transposed (the forward quantizer of a [k, n] weight)."""
  x = _x((1, rows, cols), dt, 2, gpu)
  q0, s0 = ops.quantize(x, reduce=L.REDUCE_ROWS, transpose_out=True, **KW)
  q1, s1 = ops.quantize(x, reduce=L.REDUCE_ROWS, transpose_out=True, want_other_axis_absmax=True, **KW)
  assert torch.equal(q0, q1) and torch.equal(s0, s1)
  parts = q1.other_axis_absmax
  assert parts.shape == (cols // 64, rows)
  qa = np.abs(q1[0].cpu().numpy().astype(np.int32)).T  # [rows, cols]
  for p in range(parts.shape[0]):
    np.testing.assert_array_equal(parts[p].cpu().numpy(), qa[:, 64 * p:64 * (p + 1)].max(axis=1))


def test_plans_that_cannot_leave_maxima_say_so(gpu):
  for kw in (dict(reduce=L.REDUCE_COLS, shape=(2, 64, 1024)), dict(reduce=L.REDUCE_COLS, shape=(1, 64, 256)),
             dict(reduce=L.REDUCE_ROWS, shape=(1, 100, 64)), dict(reduce=L.REDUCE_ALL, shape=(1, 128, 64))):
    x = _x(kw['shape'], 'bf16', 3, gpu)
    q, _ = ops.quantize(x, reduce=kw['reduce'], want_other_axis_absmax=True, **KW)
    assert getattr(q, 'other_axis_absmax', None) is None


@pytest.mark.parametrize('noise', [L.NOISE_NONE, L.NOISE_JAX_UNIFORM])
@pytest.mark.parametrize('producer', ['rows', 'tiles'])
def test_quantization_from_partial_maxima_gives_the_same_bits(gpu, producer, noise):
  """The second quantization of int8 values, over the other axis, with and without the maxima."""
  if producer == 'rows':
    x = _x((1, 768, 2048), 'bf16', 4, gpu)
    q, _ = ops.quantize(x, reduce=L.REDUCE_COLS, want_other_axis_absmax=True, **KW)  # [1, 768, 2048]
    again = q  # re-quantized over the rows: one scale per column
  else:
    x = _x((1, 1024, 640), 'bf16', 5, gpu)
    q, _ = ops.quantize(x, reduce=L.REDUCE_ROWS, transpose_out=True, want_other_axis_absmax=True, **KW)  # [1, 640, 1024]
    again = q  # rows of the transposed tensor are the columns of x: one scale per row of x
  parts = q.other_axis_absmax
  assert parts.shape[1] == again.shape[2]
  kw = dict(KW, reduce=L.REDUCE_ROWS, transpose_out=True, compute_dtype=torch.bfloat16, noise=noise,
            key=np.array([0, 7], np.uint32) if noise else None)
  q0, s0 = ops.quantize(again, **kw)
  q1, s1 = ops.quantize(again, absmax_partials=parts, **kw)
  assert torch.equal(q0, q1) and torch.equal(s0, s1)
  # and the workspace was left as it has to be: a plain call afterwards still agrees
  q2, s2 = ops.quantize(again, **kw)
  assert torch.equal(q0, q2) and torch.equal(s0, s2)


@pytest.mark.parametrize('dt', ['bf16', 'f32'])
def test_training_step_uses_the_maxima_and_gives_the_same_gradients(gpu, dt, monkeypatch):
  lhs = _x((384, 1024), dt, 6, gpu).requires_grad_(True)
  rhs = U.to_dev(U.rand((1024, 640), dt, 7, 0.05), dt, gpu).requires_grad_(True)
  g = U.to_dev(U.rand((384, 640), dt, 8, 1e-3), dt, gpu)
  cfg = config.set_context(config.fully_quantized(fwd_bits=8, bwd_bits=8), utils.prng_key(42), None)
  taken = []
  real = ops.quantize

  def spy(x, **kw):
    taken.append(kw.get('absmax_partials') is not None)
    return real(x, **kw)
  monkeypatch.setattr(ops, 'quantize', spy)

  def grads():
    lhs.grad = rhs.grad = None
    out, _ = cfg.dg_core(lhs, rhs, None, None, MATMUL)
    out.backward(g)
    return out.detach().clone(), lhs.grad.clone(), rhs.grad.clone()

  with_maxima = grads()
  assert sum(taken) == 2, taken  # the two residuals
  taken.clear()
  monkeypatch.setattr(aqt, 'RESIDUAL_ABSMAX', False)
  without = grads()
  assert sum(taken) == 0
  for a, b in zip(with_maxima, without):
    assert torch.equal(a, b)

"""Benchmark of the quantized dot_general hot path on one MI355X.

One step = one int8 AqtDotGeneral forward + backward (dlhs, drhs) at the LLM MLP
shape the headline metric is quoted on: lhs bf16 [8192, 4096] (0.5% outliers x20), rhs
bf16 [4096, 14336] ~N(0, 0.02), `fully_quantized(fwd_bits=8, bwd_bits=8)`:
per-token / per-channel abs-max scales, RTN forward, stochastic rounding from a
fixed PRNG key in dlhs/drhs, int32 accumulation, bf16 output.  Inputs live in HBM
before the timed region.  Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

M, K, N = 8192, 4096, 14336
OPS_PER_CONTRACTION = 2.0 * M * N * K          # 9.6207e11
OPS_PER_STEP = 3.0 * OPS_PER_CONTRACTION       # fwd + dlhs + drhs
INT8_MFMA_PEAK = 5.0e15                        # MI355X dense int8, published
MATMUL = (((1,), (0,)), ((), ()))
# HBM bytes per GEMM launch (mean of fwd, dlhs, drhs) from the FETCH_SIZE / WRITE_SIZE counter runs
# summarised in profiles/bench_int8_fwd_bwd_8192x4096x14336_hbm_traffic.txt; counters cannot be
# read from inside this process, so the figure is carried here and re-measured when the kernel changes.
GEMM_TRAFFIC_BYTES_PER_LAUNCH = 913e6


def make_inputs(device):
  import numpy as np
  import torch
  rng = np.random.default_rng(20240607)
  lhs = rng.standard_normal((M, K), dtype=np.float32)
  lhs = np.where(rng.random((M, K)) < 0.005, lhs * np.float32(20.0), lhs)
  rhs = rng.standard_normal((K, N), dtype=np.float32) * np.float32(0.02)
  g = rng.standard_normal((M, N), dtype=np.float32) * np.float32(1e-3)
  to = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(device)
  return to(lhs), to(rhs), to(g)


def cpu_baseline(seconds_budget=30.0):
  """Times the numpy oracle (a port, not the reference) on a bounded sample of the workload."""
  import numpy as np
  from oracle import aqt_ref as R
  from oracle import numerics as nm
  from oracle import prng
  m, k, n = 1024, 4096, 1792  # 1/8 of M and N, full K: same row lengths for the fwd quantizers
  rng = np.random.default_rng(1)
  lhs = nm.to_bf16(rng.standard_normal((m, k), dtype=np.float32))
  rhs = nm.to_bf16(rng.standard_normal((k, n), dtype=np.float32) * np.float32(0.02))
  g = nm.to_bf16(rng.standard_normal((m, n), dtype=np.float32) * np.float32(1e-3))
  cfg = R.set_context(R.fully_quantized(8, 8), prng.prng_key(42))
  ops = 3.0 * 2.0 * m * k * n
  times = []
  t_start = time.perf_counter()
  while True:
    t0 = time.perf_counter()
    f = R.dg_fwd(lhs, rhs, 'bf16', MATMUL, cfg)
    R.dg_bwd(g, 'bf16', MATMUL, f, cfg)
    times.append(time.perf_counter() - t0)
    if (len(times) >= 3 and time.perf_counter() - t_start > 10.0) or time.perf_counter() - t_start > seconds_budget:
      break
  best = min(times)
  cores = int(os.environ.get('OMP_NUM_THREADS', os.cpu_count() or 1))
  return {
      'value': ops / best / 1e12, 'unit': 'TOPS', 'cores': cores, 'kind': 'port',
      'sample': f'numpy oracle fwd+bwd at {m}x{k}x{n} (1/64 of the ops of one step), >= 10 s of runs, best of '
                f'{len(times)}; BLAS float64 GEMM on {cores} threads, elementwise single-thread',
  }


def decode_bench(dev):
  """Serving shapes (rhs frozen as int8, or as int4 packed two per byte, + f32 per-channel scale,
  K = 4096): device time per call of aqtx_decode_i8 (activation quantisation + contraction +
  dequantisation) and the HBM rate on the algorithmic bytes K*N (K*N/2) + 4N + 2MK + 2MN.  Weight copies rotate through >= 1 GiB so that no cache
  level can hold them; the calls are replayed from a HIP graph so that host launch overhead does
  not sit between the kernels being timed."""
  import torch
  from aqt_amd import _lib as L
  from aqt_amd import ops
  k = 4096
  rows = []
  # the pure reader on the same bytes, the same way (HIP graph replay, 1 GiB rotation): what "as fast as the
  # memory system reads this weight once" means on this box
  ceiling, _ = read_ceiling(dev, sizes=[4096 * k // 2, 4096 * k, 14336 * k // 2, 14336 * k])
  # weights in this library's serving format (MFMA fragment order, what a frozen layer keeps) and,
  # for int8, also as plain rows [n][k] (what a caller holding the reference's layout passes)
  for w_kind, layout in (('int8', 'fragments'), ('int4_packed', 'fragments'), ('int8', 'rows')):
    packed = w_kind == 'int4_packed'
    wbytes_per = 0.5 if packed else 1.0
    for n in (4096, 14336):
      ncopies = int((1 << 30) // (n * k * wbytes_per)) + 1
      if packed:
        weights = [torch.randint(0, 256, (n, k // 2), dtype=torch.uint8, device=dev) for _ in range(ncopies)]
      else:
        weights = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(ncopies)]
      w_scale = torch.rand(n, device=dev) * 1e-3 + 1e-5
      kw = dict(quant_bound=127.5, clip_bound=127.0, w_dtype=L.I4P if packed else L.I8)
      if layout == 'fragments':
        weights = [ops.tile_weight(w, kw['w_dtype']) for w in weights]
        kw['w_layout'] = L.W_FRAGMENTS
      for m in (1, 8, 32, 64):
        x = torch.randn(m, k, device=dev).to(torch.bfloat16)
        us = _graph_replay_us(lambda: [ops.decode(x, w, w_scale, **kw) for w in weights], ncopies)
        nbytes = int(k * n * wbytes_per) + 4 * n + 2 * m * k + 2 * m * n
        rows.append({'weights': w_kind, 'layout': layout, 'n': n, 'm': m, 'us_per_call': round(us, 2),
                     'GB/s': round(nbytes / us / 1e3, 1), 'frac_of_8TBps': round(nbytes / us / 1e3 / 8000.0, 3),
                     'pure_read_of_the_weight_us': ceiling[int(k * n * wbytes_per)]['us_per_read'],
                     'frac_of_pure_read': round(ceiling[int(k * n * wbytes_per)]['us_per_read'] / us, 3)})
      del weights
  return rows


def other_configs(dev):
  """The fp8 attention projection (forward+backward) and the int4-weight tiled contraction
  (forward) at their full sizes: parity-test configurations timed for reference, not the metric."""
  import torch
  from aqt_amd.v2 import aqt_dot_general as aqt
  from aqt_amd.v2 import config, tiled_dot_general, utils

  def timeit(f, n=5, w=2):
    for _ in range(w):
      f()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(n):
      f()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / n * 1e3

  out = {}
  # fp8 'bsd,dhk->bshk', per-tensor scales, e4m3 forward, e5m2 gradients with mantissa SR
  x = torch.randn(8, 4096, 4096, device=dev).to(torch.bfloat16).requires_grad_(True)
  w = (torch.randn(4096, 32, 128, device=dev) * 0.02).to(torch.bfloat16).requires_grad_(True)
  g = (torch.randn(8, 4096, 32, 128, device=dev) * 1e-3).to(torch.bfloat16)
  cfg = config.config_v4(fwd_bits='e4m3', dlhs_bits='e5m2', drhs_bits='e5m2')
  for raw in (cfg.fwd, cfg.dlhs, cfg.drhs):
    raw.dg_quantizer.lhs.calib_shared_axes = 'per_tensor'
    raw.dg_quantizer.rhs.calib_shared_axes = 'per_tensor'
  cfg = config.set_context(cfg, utils.prng_key(1), None)

  def step4():
    x.grad = None
    w.grad = None
    aqt.einsum('bsd,dhk->bshk', x, w, cfg).backward(g)

  ms = timeit(step4)
  out['fp8_einsum_bsd_dhk_fwd_bwd'] = {'ms_per_step': round(ms, 3), 'TFLOP/s': round(3 * 2 * 32768 * 4096 * 4096 / ms / 1e9, 1)}
  # the same step with the three contractions through bf16 (float32-like sums, aqtx_gemm_plan.accumulate = AQTX_ACC_F32)
  from aqt_amd import _lib as L
  from aqt_amd import ops
  fast = ops.FP8_ACCUMULATE
  try:
    ops.FP8_ACCUMULATE = L.ACC_F32
    ms = timeit(step4)
  finally:
    ops.FP8_ACCUMULATE = fast
  out['fp8_einsum_bsd_dhk_fwd_bwd_f32_sums'] = {'ms_per_step': round(ms, 3), 'TFLOP/s': round(3 * 2 * 32768 * 4096 * 4096 / ms / 1e9, 1)}
  del x, w, g
  # int4 weights / int8 activations, groups of 128 along K (tiled dot_general), forward
  lhs = torch.randn(2048, 8192, device=dev).to(torch.bfloat16)
  rhs = (torch.randn(8192, 28672, device=dev) * 0.015).to(torch.bfloat16)
  dg = config.set_context(aqt.dot_general_make(8, 4), None, None)
  tcfg = tiled_dot_general.Cfg(
      lhs=tiled_dot_general.TensorTiling([tiled_dot_general.AxisTiling(axis=1, tile_size=128)], []),
      rhs=tiled_dot_general.TensorTiling([tiled_dot_general.AxisTiling(axis=0, tile_size=128)], []))

  def step5():
    with torch.no_grad():
      tiled_dot_general.tiled_dot_general(tcfg, lhs, rhs, MATMUL, dot_general=dg)

  ms = timeit(step5)
  out['int4w_int8a_tiled128_fwd'] = {'ms_per_call': round(ms, 3), 'TOPS': round(2 * 2048 * 8192 * 28672 / ms / 1e9, 1)}
  # the same contraction as a serving layer: the int4 weight frozen once (packed two values per byte), only the
  # activations quantized per call
  from aqt_amd.v2.flax import aqt_flax
  mk = lambda mode: aqt_flax.AqtDotGeneral(
      aqt.dot_general_make(8, 4), rhs_quant_mode=mode, tiling_cfg=tcfg, use_legacy_freezer=False,
      lhs_freeze_mode=aqt_flax.FreezerMode.CALIBRATION, rhs_freeze_mode=aqt_flax.FreezerMode.CALIBRATION_AND_VALUE,
      rngs={'params': utils.prng_key(0)})
  with torch.no_grad():
    conv = mk(utils.QuantMode.CONVERT)
    conv(lhs, rhs, MATMUL, None)
    serve = mk(utils.QuantMode.SERVE)
    serve.load_variables(conv.variables())
    ms = timeit(lambda: serve(lhs, rhs, MATMUL, None))
  out['int4w_packed_frozen_tiled128_serving_fwd'] = {
      'ms_per_call': round(ms, 3), 'TOPS': round(2 * 2048 * 8192 * 28672 / ms / 1e9, 1)}
  # the same frozen layer with a handful of tokens (one wave per 16 weight rows instead of 128-row tiles of the
  # output), replayed from a HIP graph: activation quantisation + contraction; GB/s on the packed weight's bytes
  from aqt_amd.v2 import hip_graph
  few = {}
  with torch.no_grad():
    for m_few in (1, 8, 64):
      xf = lhs[:m_few].contiguous()
      graphed = hip_graph.GraphedCall(lambda a: serve(a, rhs, MATMUL, None), xf)
      us = timeit(graphed.replay, n=20, w=3) * 1e3
      few[f'm{m_few}'] = {'us_per_call': round(us, 1), 'weight_GB/s': round(8192 * 28672 / 2 / us / 1e3, 1)}
      del graphed
  out['int4w_packed_frozen_tiled128_serving_few_tokens'] = few
  del conv, serve
  del lhs, rhs
  # one decode-sized serving layer call (8 x 4096 against a frozen int8 [4096, 14336] weight): issued from Python
  # each time, and recorded once into a HIP graph and replayed (host time included in both)
  from aqt_amd.v2 import hip_graph
  xs = torch.randn(8, 4096, device=dev).to(torch.bfloat16)
  ws = (torch.randn(4096, 14336, device=dev) * 0.02).to(torch.bfloat16)
  mk8 = lambda mode: aqt_flax.AqtDotGeneral(
      config.fully_quantized(use_stochastic_rounding=False), rhs_quant_mode=mode, use_legacy_freezer=False,
      rhs_freeze_mode=aqt_flax.FreezerMode.CALIBRATION_AND_VALUE, rngs={'params': utils.prng_key(0)})
  with torch.no_grad():
    conv = mk8(utils.QuantMode.CONVERT)
    conv(xs, ws, MATMUL, None)
    serve = mk8(utils.QuantMode.SERVE)
    serve.load_variables(conv.variables())
    call = lambda a: serve(a, ws, MATMUL, None)
    graphed = hip_graph.GraphedCall(call, xs)
    out['int8_frozen_serving_layer_call_m8_4096x14336'] = {
        'eager_us_per_call': round(timeit(lambda: call(xs), n=100, w=10) * 1e3, 1),
        'hip_graph_us_per_call': round(timeit(lambda: graphed(xs), n=100, w=10) * 1e3, 1)}
  del conv, serve, graphed
  # weight-only serving (the lhs stays bf16, frozen int8 / int4 rhs [4096, 14336]): ten layer calls recorded
  # into one HIP graph, so the figure is the call's device time (the weight streamed once and converted
  # to bf16 in registers), not the gap between graph launches
  from aqt_amd.v2 import aqt_dot_general
  wo = {}
  with torch.no_grad():
    for bits in (8, 4):
      cfg = config.set_context(aqt_dot_general.dot_general_make(None, bits), None, None)
      _, (_, wq) = cfg.dg_core(xs, ws, None, None, MATMUL)
      for m_few in (1, 8, 64):
        xf = torch.randn(m_few, 4096, device=dev).to(torch.bfloat16)

        def ten(a):
          for _ in range(9):
            cfg.dg_core(a, ws, None, wq, MATMUL)
          return cfg.dg_core(a, ws, None, wq, MATMUL)[0]

        graphed = hip_graph.GraphedCall(ten, xf)
        us = timeit(graphed.replay, n=10, w=3) * 1e3 / 10
        wo[f'int{bits}_m{m_few}'] = {'us_per_call': round(us, 1), 'weight_GB/s': round(4096 * 14336 * bits / 8 / us / 1e3, 1)}
        del graphed
      del wq
    # the narrow weight of the same block (14336 -> 4096) against 64 tokens: 64-row tiles with k in slices
    wn = (torch.randn(14336, 4096, device=dev) * 0.02).to(torch.bfloat16)
    cfg = config.set_context(aqt_dot_general.dot_general_make(None, 8), None, None)
    xn = torch.randn(64, 14336, device=dev).to(torch.bfloat16)
    _, (_, wq) = cfg.dg_core(xn, wn, None, None, MATMUL)

    def ten_narrow(a):
      for _ in range(9):
        cfg.dg_core(a, wn, None, wq, MATMUL)
      return cfg.dg_core(a, wn, None, wq, MATMUL)[0]

    graphed = hip_graph.GraphedCall(ten_narrow, xn)
    us = timeit(graphed.replay, n=10, w=3) * 1e3 / 10
    wo['int8_m64_14336x4096'] = {'us_per_call': round(us, 1), 'weight_GB/s': round(4096 * 14336 / us / 1e3, 1)}
    del graphed, wq, wn, xn
  out['weight_only_frozen_serving_few_tokens_4096x14336'] = wo
  del xs, ws
  # quantized ragged_dot (mixture of experts): 8192 tokens routed to 8 experts [4096, 14336], uneven groups,
  # forward, with the expert weights quantized on the fly (the reference's ragged_dot does the same) and
  # with the contraction alone (operands already int8)
  from aqt_amd import ops
  from aqt_amd.v2 import aqt_ragged_dot
  tokens, experts, kk, nn = 8192, 8, 4096, 14336
  x = torch.randn(tokens, kk, device=dev).to(torch.bfloat16)
  w = (torch.randn(experts, kk, nn, device=dev) * 0.02).to(torch.bfloat16)
  sizes = torch.tensor([1500, 700, 1024, 0, 2100, 900, 1200, 768], dtype=torch.int32, device=dev)

  def step6():
    with torch.no_grad():
      aqt_ragged_dot.ragged_dot(x, w, sizes)

  ms = timeit(step6)
  xq = torch.randint(-127, 128, (1, tokens, kk), dtype=torch.int8, device=dev)
  wq = torch.randint(-127, 128, (experts, nn, kk), dtype=torch.int8, device=dev)
  offs = torch.zeros(experts + 1, dtype=torch.int32, device=dev)
  offs[1:] = torch.cumsum(sizes, 0)
  ms_gemm = timeit(lambda: ops.gemm(xq, wq, row_scale=None, col_scale=None, out_dtype=torch.int32, group_offsets=offs))
  gop = 2.0 * tokens * kk * nn / 1e9
  out['ragged_dot_int8_fwd_8192tok_8experts'] = {
      'ms_per_call': round(ms, 3), 'TOPS': round(gop / ms, 1),
      'contraction_only_ms': round(ms_gemm, 3), 'contraction_only_TOPS': round(gop / ms_gemm, 1)}
  del x, w, xq, wq
  # emulated fp4 (e2m1 with subnormals) in a bf16 container, 8192 x 14336: one read and one write per element
  from aqt_amd.v2.numerics import fp_numerics
  t = torch.randn(8192, 14336, device=dev).to(torch.bfloat16)
  key = utils.prng_key(3)
  ms_rn = timeit(lambda: fp_numerics.fp_round(t, cfg=fp_numerics.e2m1_ocp, key=None, stochastic_rounding=False))
  ms_sr = timeit(lambda: fp_numerics.fp_round(t, cfg=fp_numerics.e2m1_ocp, key=key, stochastic_rounding=True))
  gb = 2 * 2 * t.numel() / 1e9
  out['fp_round_e2m1_bf16_8192x14336'] = {
      'nearest_ms': round(ms_rn, 3), 'nearest_GB/s': round(gb / ms_rn * 1e3, 1),
      'stochastic_ms': round(ms_sr, 3), 'stochastic_GB/s': round(gb / ms_sr * 1e3, 1)}
  del t
  # quantized conv_general_dilated forward (NHWC input [32, 56, 56, 128], 3x3 kernel to 128 features, SAME): per
  # batch-element input scale, per-feature kernel scale, window gather + int8 contraction with fused dequantisation
  from aqt_amd.v2 import aqt_conv_general
  xc = torch.randn(32, 56, 56, 128, device=dev).to(torch.bfloat16)
  kc = (torch.randn(3, 3, 128, 128, device=dev) * 0.05).to(torch.bfloat16)
  conv = aqt_conv_general.make_conv_general_dilated(aqt_conv_general.conv_general_dilated_make(2, 8, 8))
  dnc = aqt_conv_general.flax_conv_dimension_numbers(xc.shape)
  with torch.no_grad():
    call = lambda a: conv(a, kc, (1, 1), 'SAME', dimension_numbers=dnc)
    ms = timeit(lambda: call(xc))
    graphed = hip_graph.GraphedCall(call, xc)
    ms_graph = timeit(graphed.replay, n=20, w=3)
  gop = 2.0 * 32 * 56 * 56 * 9 * 128 * 128 / 1e9
  out['conv_int8_fwd_32x56x56x128_k3x3_128'] = {
      'ms_per_call': round(ms, 3), 'TOPS': round(gop / ms, 1),
      'hip_graph_ms_per_call': round(ms_graph, 3), 'hip_graph_TOPS': round(gop / ms_graph, 1)}
  del graphed, xc, kc
  # the reference's own small case: a two-layer MLP block, x f32 [4096, 512], Dense 512 -> 2048, ReLU,
  # Dense 2048 -> 512, fully_quantized(8, 8) with stochastic rounding in the backward pass, forward + backward
  # issued from Python (host time included: at this size the step is bound by it, not by the kernels)
  xm = torch.randn(4096, 512, device=dev, requires_grad=True)
  w1 = (torch.randn(512, 2048, device=dev) / 512 ** 0.5).requires_grad_(True)
  w2 = (torch.randn(2048, 512, device=dev) / 2048 ** 0.5).requires_grad_(True)
  gm = torch.randn(4096, 512, device=dev) / (4096 * 512)
  mlp_cfg = config.fully_quantized(fwd_bits=8, bwd_bits=8)
  k1, k2 = utils.prng_key(1), utils.prng_key(2)

  def step_mlp():
    h = config.set_context(mlp_cfg, k1, None)(xm, w1, MATMUL)
    y = config.set_context(mlp_cfg, k2, None)(torch.relu(h), w2, MATMUL)
    y.backward(gm)
    xm.grad = w1.grad = w2.grad = None

  ms = timeit(step_mlp, n=30, w=5)
  # the same step recorded once into a HIP graph: the keys live in device tensors (their fan-out is a kernel,
  # the quantizers read them from device memory), so every replay draws the noise of the keys it finds there
  import numpy as np
  kd1 = torch.from_numpy(np.asarray(k1, dtype=np.uint32).view(np.int32).copy()).to(dev)
  kd2 = torch.from_numpy(np.asarray(k2, dtype=np.uint32).view(np.int32).copy()).to(dev)

  def step_mlp_recorded():
    xm.grad = w1.grad = w2.grad = None
    h = config.set_context(mlp_cfg, kd1, None)(xm, w1, MATMUL)
    y = config.set_context(mlp_cfg, kd2, None)(torch.relu(h), w2, MATMUL)
    y.backward(gm)
    return y

  graphed = hip_graph.GraphedStep(step_mlp_recorded)
  ms_graph = timeit(graphed.replay, n=50, w=5)
  mlp_gop = 3 * 2 * 2 * 4096 * 512 * 2048 / 1e9
  out['mlp_block_f32_4096x512_2048_512_fwd_bwd'] = {
      'ms_per_step_from_python': round(ms, 3), 'TOPS': round(mlp_gop / ms, 1),
      'hip_graph_ms_per_step': round(ms_graph, 3), 'hip_graph_TOPS': round(mlp_gop / ms_graph, 1)}
  del graphed, xm, w1, w2, gm
  # the configurations whose contraction is a float one, forward call at 4096^3 bf16, ms per call from Python
  out['float_contraction_modes_fwd_4096x4096x4096_ms'] = float_modes(dev)
  return out


def float_modes(dev, calls=10, warm=3, only=None):
  """Forward calls of the configurations that contract in float (aqt_dot_general.py:843-958) at 4096 x 4096 x 4096,
  bf16, int8 numerics, issued from Python: fake quantization with contraction-axis and with remaining-axis
  calibration, a fake-quantized lhs against an int8 rhs dequantized at the output, the lhs scale applied to the
  rhs (OTHER_INPUT), integers held in the float dtype, an unquantized lhs against a freshly quantized rhs; the
  default int8 path beside them.  Returns {name: ms per call}."""
  import torch
  from aqt_amd.v2 import aqt_dot_general as aqt
  m = k = n = 4096
  lhs = torch.randn(m, k, device=dev).to(torch.bfloat16)
  rhs = (torch.randn(k, n, device=dev) * 0.02).to(torch.bfloat16)
  out_m, this_m, other_m = aqt.DequantMode.OUTPUT, aqt.DequantMode.THIS_INPUT, aqt.DequantMode.OTHER_INPUT
  ca, ra = aqt.CalibrationMode.CONTRACTING_AXIS, aqt.CalibrationMode.REMAINING_AXIS

  def make(lbits=8, rbits=8, lmode=out_m, rmode=out_m, lcal=ca, rcal=ca, held=False):
    raw = aqt.dot_general_raw_make(lbits, rbits, initialize_calibration=False)
    raw.lhs.dequant_mode, raw.rhs.dequant_mode = lmode, rmode
    raw.lhs.calibration_mode, raw.rhs.calibration_mode = lcal, rcal
    if (lmode, rmode) != (out_m, out_m) or held:
      raw.dg_accumulator_dtype = None
    if held:
      raw.dg_quantizer.lhs.numerics.dtype = raw.dg_quantizer.rhs.numerics.dtype = None
    raw.dg_quantizer.init_calibration()
    return raw

  cfgs = {
      'int8_default': make(),
      'fake_quant': make(lmode=this_m, rmode=this_m),
      'fake_quant_float_held': make(lmode=this_m, rmode=this_m, held=True),
      'fake_quant_remaining_axis': make(lmode=this_m, rmode=this_m, lcal=ra, rcal=ra),
      'lhs_scale_into_rhs': make(lmode=other_m, rmode=this_m, lcal=ra, rcal=ra),
      'fake_quant_lhs_int8_rhs': make(lmode=this_m),
      'float_lhs_int8_rhs': make(lbits=None),
  }
  res = {}
  with torch.no_grad():
    for name, raw in cfgs.items():
      if only is not None and name != only:
        continue
      for _ in range(warm):
        raw(lhs, rhs, None, None, MATMUL)
      torch.cuda.synchronize()
      t0 = time.perf_counter()
      for _ in range(calls):
        raw(lhs, rhs, None, None, MATMUL)
      torch.cuda.synchronize()
      res[name] = round((time.perf_counter() - t0) / calls * 1e3, 3)
  return res


def _graph_replay_us(run, ncalls, reps=5):
  """Device time per call of the `ncalls` launches `run` makes, replayed `reps` times from one HIP graph."""
  import torch
  run()
  torch.cuda.synchronize()
  side = torch.cuda.Stream()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.stream(side):
    run()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
      keep = run()
  torch.cuda.synchronize()
  graph.replay()
  torch.cuda.synchronize()
  a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  a.record()
  for _ in range(reps):
    graph.replay()
  b.record()
  torch.cuda.synchronize()
  us = a.elapsed_time(b) * 1e3 / (reps * ncalls)
  del graph, keep
  return us


# launch shapes of the pure reader that came out on top of the full sweep (read_ceiling(full=True)) at the
# serving weights' sizes: (workgroups, 16-byte loads in flight per lane, cache policy)
_READER_SHAPES = ((512, 4, 2), (512, 4, 3), (1024, 2, 2), (512, 8, 2), (256, 8, 2), (1024, 4, 2))


def read_ceiling(dev, full=False, sizes=None):
  """What this box's memory system delivers to a kernel that only reads a buffer once (aqtx_read_probe: each
  wave load one contiguous KiB, one checksum word per workgroup, nothing else).  Two figures per launch shape:
  'span_us' = last workgroup's end minus first workgroup's start on the device clock (median of 7 launches, no
  launch overhead in it), and 'us_per_read' = back-to-back launches replayed from a HIP graph, the way
  decode_bench times the serving calls; buffers rotate through >= 1 GiB either way.  full: the sweep over
  sizes (the two int8 serving weights, 256 MiB, 1 GiB), workgroups per CU (one chunk per workgroup, or 1 / 2 / 4 /
  8 / 16 persistent ones), loads in flight per lane (2..16 x 16 bytes) and cache policy; otherwise the few shapes
  that won that sweep, at the given sizes.  Returns {bytes: best row} and all rows."""
  import torch
  from aqt_amd import ops
  cus = torch.cuda.get_device_properties(dev).multi_processor_count
  if sizes is None:
    sizes = [4096 * 4096, 14336 * 4096, 256 << 20, 1 << 30] if full else [4096 * 4096, 14336 * 4096]
  if full:
    shapes = [(w * cus if w else 0, u, pol) for pol in (0, 2, 3) for u in (2, 4, 8, 16) for w in (0, 1, 2, 4, 8, 16)]
  else:
    shapes = list(_READER_SHAPES)
  out_words = torch.zeros(65536, dtype=torch.int32, device=dev)
  stamps = torch.zeros(2 * 65536, dtype=torch.int64, device=dev)
  rows, best = [], {}
  for nbytes in sizes:
    ncopies = max(2, (1 << 30) // nbytes + 1)
    pool = torch.randint(-128, 128, (ncopies * nbytes,), dtype=torch.int8, device=dev)
    bufs = [pool[i * nbytes:(i + 1) * nbytes] for i in range(ncopies)]
    for wg, u, pol in shapes:
      nwg = ops.read_probe_workgroups(nbytes, wg, u)
      if nwg > 65536 or (wg and nwg < wg):
        continue
      kw = dict(workgroups=wg, loads_in_flight=u, cache_policy=pol)
      spans = []
      for i in range(8):
        ops.read_probe(bufs[i % ncopies], out_words, stamps=stamps, **kw)
        torch.cuda.synchronize()
        spans.append(ops.read_probe_span_us(stamps, nwg))
      span = sorted(spans[1:])[3]
      us = _graph_replay_us(lambda: [ops.read_probe(b, out_words, **kw) for b in bufs], ncopies, reps=3)
      row = {'bytes': nbytes, 'workgroups': nwg, 'per_cu': round(nwg / cus, 2) if wg else 'one chunk each',
             'loads_in_flight': u, 'cache_policy': pol, 'span_us': round(span, 2), 'span_TB/s': round(nbytes / span / 1e6, 2),
             'us_per_read': round(us, 2), 'TB/s': round(nbytes / us / 1e6, 2)}
      rows.append(row)
      if nbytes not in best or us < best[nbytes]['us_per_read']:
        best[nbytes] = row
    del bufs, pool
  return best, rows


def decode_probe(dev, calibration_copy=False):
  """A few eager serving calls per shape (int8 weight in fragment order, n in {4096, 14336},
  m in {1, 8, 64}, weights rotated through 1 GiB) for counter and kernel-trace runs of the
  serving kernels, plus one read of each weight size by aqtx_read_probe."""
  import torch
  from aqt_amd import _lib as L
  from aqt_amd import ops
  if calibration_copy:
    src = torch.ones(64 << 20, dtype=torch.int32, device=dev)
    torch.neg(src, out=torch.empty_like(src))  # 256 MiB in, 256 MiB out
    del src
  k = 4096
  for n in (4096, 14336):
    ncopies = (1 << 30) // (n * k) + 1
    raw = [torch.randint(-127, 128, (n, k), dtype=torch.int8, device=dev) for _ in range(ncopies)]
    weights = [ops.tile_weight(w, L.I8) for w in raw]
    w_scale = torch.rand(n, device=dev) * 1e-3 + 1e-5
    for w in raw:
      ops.read_probe(w)
    for m in (1, 8, 64):
      x = torch.randn(m, k, device=dev).to(torch.bfloat16)
      for w in weights:
        ops.decode(x, w, w_scale, quant_bound=127.5, clip_bound=127.0, w_layout=L.W_FRAGMENTS)
    torch.cuda.synchronize()
    del raw, weights
  print(json.dumps({'decode_probe': 'done'}))


def gemm_probe(dev, data, reps=10):
  """The three contractions of a step on their own, on synthetic int8 operands of a chosen value
  distribution (the MFMA rate of this part depends on the operand values: the chip lowers its
  clock when more datapath bits toggle), next to the vendor library's int8 GEMM (torch._int_mm,
  raw int32 output) on the same operands.  For counter runs (rocprofv3 --pmc) and the
  data-dependence table; prints one JSON line."""
  import torch
  from aqt_amd import ops
  gens = {
      'zeros': lambda s: torch.zeros(s, dtype=torch.int8, device=dev),
      'normal25': lambda s: (torch.randn(s, device=dev) * 25).clamp(-127, 127).round().to(torch.int8),
      'uniform': lambda s: torch.randint(-127, 128, s, dtype=torch.int8, device=dev),
  }
  gen = gens[data]

  def timed(f):
    for _ in range(3):
      f()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(reps):
      f()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / reps

  rows = {}
  for shape, (m, n, k) in (('fwd', (M, N, K)), ('dlhs', (M, K, N)), ('drhs', (K, N, M))):
    a, b = gen((1, m, k)), gen((1, n, k))
    rs, cs = torch.rand(1, m, device=dev), torch.rand(1, n, device=dev)
    ms = timed(lambda: ops.gemm(a, b, row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16))
    # the library takes the second operand [k, n]: the rows of b viewed transposed (k contiguous in both
    # operands, as this library reads them), and a [k, n] copy
    ms_lib = timed(lambda: torch._int_mm(a[0], b[0].t()))
    bt = b[0].t().contiguous()
    ms_lib_kn = timed(lambda: torch._int_mm(a[0], bt))
    ops_ = 2.0 * m * n * k
    rows[shape] = {'m': m, 'n': n, 'k': k, 'aqtx_gemm_i8_us': round(ms * 1e3, 1), 'aqtx_TOPS': round(ops_ / ms / 1e9),
                   'library_int_mm_us': round(ms_lib * 1e3, 1), 'library_TOPS': round(ops_ / ms_lib / 1e9),
                   'library_int_mm_kn_copy_us': round(ms_lib_kn * 1e3, 1), 'library_kn_copy_TOPS': round(ops_ / ms_lib_kn / 1e9)}
    del a, b, bt
  print(json.dumps({'gemm_probe': data, 'reps': reps, 'shapes': rows}))


def prefill_probe_cold(dev):
  """prefill_probe's two int8 columns with a different weight every call: the calls of one HIP-graph replay walk
  through about 1 GiB of distinct weights (24 or 18 of them), so that every weight comes from HBM, as the
  weights of successive layers do, next to the same calls against one weight that stays in the memory-side cache.
  The `fragments` columns read the weight in the serving kernels' fragment order (aqtx_tile_weight), which is what
  a frozen weight of the layer API is kept in."""
  import torch
  from aqt_amd import ops, _lib as L

  def t(f, calls):
    return round(_graph_replay_us(f, calls, reps=3), 1)

  def ints(shape):
    return (torch.randn(shape, device=dev) * 25).clamp(-127, 127).round().to(torch.int8)

  for n, k in ((4096, 4096), (14336, 4096), (4096, 14336)):
    nw = min(24, max(2, (1 << 30) // (n * k)))
    ws = [ints((1, n, k)) for _ in range(nw)]
    frs = [ops.tile_weight(w[0], L.I8) for w in ws]
    cs = torch.rand(1, n, device=dev) * 0.01 + 1e-4
    for m in (128, 256, 512, 1024, 2048):
      a = ints((1, m, k))
      rs = torch.rand(1, m, device=dev) * 0.01 + 1e-4
      kw = dict(row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16, scale_dtype=torch.bfloat16)
      print(json.dumps({
          'prefill_probe_cold': 'us per call', 'm': m, 'n': n, 'k': k, 'weights_walked': nw,
          'aqtx_gemm_i8_from_hbm': t(lambda: [ops.gemm(a, w, **kw) for w in ws], nw),
          'aqtx_gemm_i8_fragments_from_hbm': t(lambda: [ops.gemm(a, f, b_layout=L.W_FRAGMENTS, **kw) for f in frs], nw),
          'vendor_int_mm_from_hbm': t(lambda: [torch._int_mm(a[0], w[0].t()) for w in ws], nw),
          'aqtx_gemm_i8_one_weight': t(lambda: [ops.gemm(a, ws[0], **kw) for _ in range(10)], 10),
          'aqtx_gemm_i8_fragments_one_weight': t(lambda: [ops.gemm(a, frs[0], b_layout=L.W_FRAGMENTS, **kw) for _ in range(10)], 10),
          'vendor_int_mm_one_weight': t(lambda: [torch._int_mm(a[0], ws[0][0].t()) for _ in range(10)], 10)}), flush=True)
      del a
    del ws, frs


def prefill_probe(dev, shapes=False):
  """Contractions of prefill-sized serving calls (128..4096 rows against the 4096 x 14336 MLP weights and a
  4096 x 4096 one), device time per call replayed from a HIP graph, microseconds: aqtx_gemm_i8 (int8 operands
  drawn from round(25 * normal), bf16 output with both scales fused, the library's own choice of kernel) next to
  the vendor int8 GEMM (torch._int_mm, raw int32 output), and aqtx_gemm_weight_only (bf16 rows, int8 weight)
  next to the vendor bf16 product on a bf16 copy of the weight.  With `shapes`, also every tile shape of the
  kernel for few output tiles forced through plan->tuning (their results are compared bit for bit with the
  library's choice).  Prints one JSON line per shape."""
  import torch
  from aqt_amd import ops

  def t(f, calls=10):
    return round(_graph_replay_us(lambda: [f() for _ in range(calls)], calls, reps=3), 1)

  def ints(shape):
    return (torch.randn(shape, device=dev) * 25).clamp(-127, 127).round().to(torch.int8)

  forced = (('tiles128', 128), ('ring128', 129), ('ring64x128', 130), ('ring64', 131), ('ring128x256', 132), ('ring64pair', 133), ('ring64x128pair', 134)) if shapes else ()
  saved = ops.GEMM_TUNING
  for n, k in ((4096, 4096), (14336, 4096), (4096, 14336)):
    b = ints((1, n, k))
    bt = b[0].t()  # the vendor int8 GEMM takes the second operand [k, n]: the same rows, viewed transposed
    bf = b[0].to(torch.bfloat16)
    cs = torch.rand(1, n, device=dev) * 0.01 + 1e-4
    for m in (128, 256, 512, 1024, 2048, 4096):
      a = ints((1, m, k))
      x = torch.randn(1, m, k, device=dev).to(torch.bfloat16)
      rs = torch.rand(1, m, device=dev) * 0.01 + 1e-4
      kw = dict(row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16, scale_dtype=torch.bfloat16)
      ops.GEMM_TUNING = saved
      ref = ops.gemm(a, b, **kw)
      row = {'prefill_probe': 'us per call', 'm': m, 'n': n, 'k': k, 'aqtx_gemm_i8': t(lambda: ops.gemm(a, b, **kw)),
             'vendor_int_mm': t(lambda: torch._int_mm(a[0], bt))}
      for name, tuning in forced:
        ops.GEMM_TUNING = tuning
        out = ops.gemm(a, b, k_split=1, **kw)
        assert torch.equal(out, ref), (name, m, n, k)
        row[name] = t(lambda: ops.gemm(a, b, k_split=1, **kw))
      ops.GEMM_TUNING = saved
      row['aqtx_gemm_weight_only'] = t(lambda: ops.gemm_weight_only(x, b, cs))
      row['vendor_bf16_on_a_copy'] = t(lambda: torch.matmul(x[0], bf.t()))
      print(json.dumps(row), flush=True)
      del a, x
    del b, bt, bf


def power_probe(dev, seconds=8.0):
  """Socket power and shader clock, sampled from the box's SMI tool (amd-smi) by a thread of this
  process while the forward contraction (8192 x 14336 x 4096) runs back to back for `seconds` per operand value
  distribution: the evidence behind 'the clock falls with the operand values under the power cap'.  Prints one
  JSON line; where no tool answers an ordinary user, the samples are empty and the line says so."""
  import re
  import shutil
  import subprocess
  import threading
  import torch
  from aqt_amd import ops
  tool = shutil.which('amd-smi') or '/opt/rocm/bin/amd-smi'
  cap = None

  def sample():
    """(watts, mean MHz over the XCDs) or None."""
    try:
      out = subprocess.run([tool, 'metric', '-g', '0', '-p', '-c', '--json'], capture_output=True, text=True, timeout=10).stdout
      card = json.loads(out)
      card = (card['gpu_data'] if isinstance(card, dict) else card)[0]
      watts = card['power']['socket_power']['value']
      clks = [v['clk']['value'] for k, v in card['clock'].items() if k.startswith('gfx_') and isinstance(v['clk']['value'], (int, float))]
      return (float(watts) if isinstance(watts, (int, float)) else None), (sum(clks) / len(clks) if clks else None)
    except Exception:
      return None

  try:  # the package power limit, from the older tool (it answers an ordinary user)
    out = subprocess.run([shutil.which('rocm-smi') or '/opt/rocm/bin/rocm-smi', '-d', '0', '--showmaxpower', '--json'],
                         capture_output=True, text=True, timeout=10).stdout
    cap = next((float(v) for k, v in next(iter(json.loads(out).values())).items() if re.match(r'^[0-9.]+$', str(v))), None)
  except Exception:
    pass
  gens = {
      'zeros': lambda s: torch.zeros(s, dtype=torch.int8, device=dev),
      'normal25': lambda s: (torch.randn(s, device=dev) * 25).clamp(-127, 127).round().to(torch.int8),
  }
  rows = {'idle': {'samples': [sample() for _ in range(3)]}}
  for kind, gen in gens.items():
    a, b = gen((1, M, K)), gen((1, N, K))
    rs, cs = torch.rand(1, M, device=dev), torch.rand(1, N, device=dev)
    f = lambda: ops.gemm(a, b, row_scale=rs, col_scale=cs, out_dtype=torch.bfloat16)
    for _ in range(5):
      f()
    torch.cuda.synchronize()
    samples, stop = [], threading.Event()

    def poll():
      while not stop.is_set():
        r = sample()
        if r is not None:
          samples.append(r)

    th = threading.Thread(target=poll)
    th.start()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0, calls = time.perf_counter(), 0
    e0.record()
    while time.perf_counter() - t0 < seconds:
      for _ in range(50):
        f()
      calls += 50
      torch.cuda.synchronize()
    e1.record()
    torch.cuda.synchronize()
    stop.set()
    th.join()
    us = e0.elapsed_time(e1) * 1e3 / calls
    watts = [w for w, _ in samples if w is not None]
    mhz = [c for _, c in samples if c is not None]
    rows[kind] = {'us_per_launch': round(us, 1), 'TOPS': round(2.0 * M * N * K / us / 1e6), 'samples': len(samples),
                  'socket_power_W_mean': round(sum(watts) / len(watts), 1) if watts else None,
                  'socket_power_W_max': max(watts) if watts else None,
                  'sclk_MHz_mean': round(sum(mhz) / len(mhz)) if mhz else None,
                  'sclk_MHz_min': min(mhz) if mhz else None, 'sclk_MHz_max': max(mhz) if mhz else None}
    del a, b
  print(json.dumps({'power_probe': 'aqtx_gemm_i8 8192x14336x4096 back to back, SMI samples from a thread', 'tool': tool,
                    'power_cap_W': cap, 'rows': rows}))


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument('--gpus', type=int, default=1)
  ap.add_argument('--steps', type=int, default=20)
  ap.add_argument('--warmup', type=int, default=3)
  ap.add_argument('--no-cpu-baseline', action='store_true')
  ap.add_argument('--no-decode', action='store_true', help='skip the serving-shape (decode) measurements')
  ap.add_argument('--no-other-configs', action='store_true',
                  help='skip the fp8 einsum and int4-weight tiled timings')
  ap.add_argument('--calibration-copy', action='store_true',
                  help='also launch one elementwise kernel that reads and writes 256 MiB, as the '
                       'known-size reference for FETCH_SIZE / WRITE_SIZE counter runs')
  ap.add_argument('--gemm-probe', choices=['zeros', 'normal25', 'uniform'], default=None,
                  help='only run the three int8 contractions of a step on operands of this value '
                       'distribution (and the vendor int8 GEMM beside them) and exit')
  ap.add_argument('--decode-probe', action='store_true',
                  help='only issue a few serving calls per shape (for rocprofv3 runs) and exit')
  ap.add_argument('--prefill-probe', choices=['library', 'shapes', 'cold'], default=None,
                  help='only time prefill-sized contractions (128..4096 rows against the MLP weights) next to the vendor '
                       "GEMMs and exit; 'shapes' adds every tile shape of the kernel for few output tiles, 'cold' walks "
                       "through 1 GiB of distinct weights instead")
  ap.add_argument('--power-probe', action='store_true',
                  help='only run the forward contraction back to back on all-zero and on quantized-normal operands while '
                       'sampling socket power and shader clock from the SMI tool, and exit')
  ap.add_argument('--float-modes-probe', default=None, metavar='NAME',
                  help="only issue 13 forward calls of one float-contraction configuration (a key of float_modes(), or "
                       "'all') at 4096^3 bf16, print ms per call, and exit (for rocprofv3 runs)")
  ap.add_argument('--read-ceiling', action='store_true',
                  help='only sweep a pure reader over buffer sizes and launch shapes (what the memory system delivers '
                       'to a single pass over the serving weights and over 256 MiB / 1 GiB) and exit')
  args = ap.parse_args()
  if args.gpus != 1:
    print('bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)',
          file=sys.stderr)
    sys.exit(2)

  import torch
  from aqt_amd import ops
  from aqt_amd.v2 import config, utils

  if not torch.cuda.is_available():
    print('bench.py needs a GPU', file=sys.stderr)
    sys.exit(1)
  dev = torch.device('cuda:0')
  if args.gemm_probe is not None:
    gemm_probe(dev, args.gemm_probe)
    return
  if args.prefill_probe == 'cold':
    prefill_probe_cold(dev)
    return
  if args.prefill_probe is not None:
    prefill_probe(dev, shapes=args.prefill_probe == 'shapes')
    return
  if args.power_probe:
    power_probe(dev)
    return
  if args.float_modes_probe is not None:
    print(json.dumps(float_modes(dev, only=None if args.float_modes_probe == 'all' else args.float_modes_probe)))
    return
  if args.read_ceiling:
    best, rows = read_ceiling(dev, full=True)
    for r in rows:
      print(json.dumps(r))
    print(json.dumps({'read_ceiling': 'best launch shape per size (back-to-back launches from a HIP graph, 1 GiB rotation)',
                      'best': [best[b] for b in sorted(best)]}))
    return
  if args.decode_probe:
    decode_probe(dev, args.calibration_copy)
    return
  lhs, rhs, g = make_inputs(dev)
  lhs.requires_grad_(True)
  rhs.requires_grad_(True)
  cfg = config.set_context(config.fully_quantized(fwd_bits=8, bwd_bits=8), utils.prng_key(42), None)

  def step():
    lhs.grad = None
    rhs.grad = None
    out, _ = cfg.dg_core(lhs, rhs, None, None, MATMUL)
    out.backward(g)
    return out

  if args.calibration_copy:
    src = torch.ones(64 << 20, dtype=torch.int32, device=dev)
    torch.neg(src, out=torch.empty_like(src))  # 256 MiB in, 256 MiB out
    del src
  for _ in range(args.warmup):
    step()
  torch.cuda.synchronize()
  with ops.KernelTimer('gemm') as timer:
    t0 = time.perf_counter()
    for _ in range(args.steps):
      step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
  ms_per_step = elapsed / args.steps * 1e3
  gemm_ms = timer.mean_ms()
  achieved = OPS_PER_CONTRACTION / (gemm_ms * 1e-3) / 1e12

  line = {
      'metric': 'int8 dot_general TOPS @8192x4096x14336 (fwd+bwd)',
      'value': OPS_PER_STEP / (ms_per_step * 1e-3) / 1e12,
      'unit': 'TOPS',
      'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': ms_per_step,
      'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
      'dtype': 'int8', 'data': 'synthetic',
      'config': {'workload': 'configs[1]: int8 dot_general fwd+bwd, lhs bf16 [8192,4096] x rhs bf16 '
                             '[4096,14336], fully_quantized(8,8), SR key 42, bf16 out',
                 'pct_of_int8_mfma_peak': 100.0 * OPS_PER_STEP / (ms_per_step * 1e-3) / INT8_MFMA_PEAK},
      'roofline': {'bound': 'mfma', 'kernel': 'gemm_kernel<MmaI8, ...>', 'achieved': achieved,
                   'peak': INT8_MFMA_PEAK / 1e12, 'unit': 'TFLOP/s',
                   'frac': achieved * 1e12 / INT8_MFMA_PEAK, 'traffic': GEMM_TRAFFIC_BYTES_PER_LAUNCH,
                   'launch_ms': gemm_ms, 'launches_timed': len(timer.pairs)},
  }
  if not args.no_decode:
    line['decode'] = {'kernel': 'aqtx_decode_i8 (m <= 2: decode_fused_kernel; m >= 3: decode_tile_kernel, its first workgroups quantizing the tokens against a weight of 24 MiB or more and up to 32 tokens, else behind decode_quant_kernel)',
                      'k': 4096,
                      'timing': 'HIP graph replay, weights rotated through 1 GiB', 'shapes': decode_bench(dev)}
  if not args.no_other_configs:
    del lhs, rhs, g
    torch.cuda.empty_cache()
    line['other_configs'] = other_configs(dev)
  if not args.no_cpu_baseline:
    line['cpu_baseline'] = cpu_baseline()
  print(json.dumps(line))


if __name__ == '__main__':
  main()

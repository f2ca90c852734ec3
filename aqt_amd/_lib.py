"""ctypes binding of libaqtx.so (see include/aqtx.h for the contract).

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# AQTX_LIB_PATH points at another build of the same C-ABI (kernel experiments).
LIB_PATH = os.environ.get('AQTX_LIB_PATH') or os.path.join(_HERE, 'lib', 'libaqtx.so')

# element types (include/aqtx.h)
F32, BF16, I8, I4, E4M3, E5M2, I32, I4P = range(8)
REDUCE_COLS, REDUCE_ROWS, REDUCE_ALL, REDUCE_ALL_BATCH = range(4)
NOISE_NONE, NOISE_JAX_UNIFORM, NOISE_CUSTOM1, NOISE_FP8_MANTISSA = range(4)
PRESCALE_NONE, PRESCALE_PER_ROW, PRESCALE_PER_COL = range(3)
SCALE_ROW_THEN_COL, SCALE_COL_THEN_ROW = range(2)
W_ROWS, W_FRAGMENTS = range(2)
K_NATURAL, K_EVEN_ODD8 = range(2)
ACC_FAST, ACC_F32 = range(2)
FACTOR_ROWS, FACTOR_COLS = range(2)


class QuantPlan(ctypes.Structure):
  _fields_ = [
      ('in_dtype', ctypes.c_int32), ('compute_dtype', ctypes.c_int32),
      ('scale_dtype', ctypes.c_int32), ('out_dtype', ctypes.c_int32),
      ('batch', ctypes.c_int64), ('rows', ctypes.c_int64), ('cols', ctypes.c_int64),
      ('reduce', ctypes.c_int32), ('transpose_out', ctypes.c_int32),
      ('group', ctypes.c_int64),
      ('quant_bound', ctypes.c_float), ('clip_bound', ctypes.c_float),
      ('noise', ctypes.c_int32), ('partitionable', ctypes.c_int32),
      ('key', ctypes.c_uint32 * 2),
      ('noise_stride_batch', ctypes.c_int64), ('noise_stride_row', ctypes.c_int64),
      ('noise_stride_col', ctypes.c_int64), ('noise_total', ctypes.c_int64),
      ('prescale', ctypes.c_int32), ('scale_given', ctypes.c_int32),
      ('prescale_stride_batch', ctypes.c_int64),
      ('scale_typed', ctypes.c_void_p),
      ('workspace_zeroed', ctypes.c_int32),
      ('key_device', ctypes.c_void_p),
      ('out_k_order', ctypes.c_int32),
      ('other_axis_absmax', ctypes.c_void_p),
      ('absmax_partials', ctypes.c_void_p), ('absmax_parts', ctypes.c_int64),
  ]


class ScalePlan(ctypes.Structure):
  _fields_ = [
      ('in_dtype', ctypes.c_int32), ('out_dtype', ctypes.c_int32),
      ('batch', ctypes.c_int64), ('rows', ctypes.c_int64), ('cols', ctypes.c_int64),
      ('factors', ctypes.c_int32),
      ('factor_axis', ctypes.c_int32 * 2), ('factor_dtype', ctypes.c_int32 * 2),
      ('factor_recast', ctypes.c_int32 * 2),
      ('factor_stride_b', ctypes.c_int64 * 2),
      ('factor_reciprocal', ctypes.c_int32 * 2),
      ('finish_clip', ctypes.c_float), ('finish_round', ctypes.c_int32),
  ]


class GemmPlan(ctypes.Structure):
  _fields_ = [
      ('batch', ctypes.c_int64), ('m', ctypes.c_int64), ('n', ctypes.c_int64), ('k', ctypes.c_int64),
      ('lda', ctypes.c_int64), ('ldb', ctypes.c_int64), ('ldc', ctypes.c_int64),
      ('stride_a', ctypes.c_int64), ('stride_b', ctypes.c_int64), ('stride_c', ctypes.c_int64),
      ('a_dtype', ctypes.c_int32), ('b_dtype', ctypes.c_int32),
      ('out_dtype', ctypes.c_int32), ('dequant_dtype', ctypes.c_int32),
      ('row_scale_dtype', ctypes.c_int32), ('col_scale_dtype', ctypes.c_int32),
      ('scale_order', ctypes.c_int32),
      ('row_scale_stride_b', ctypes.c_int64), ('col_scale_stride_b', ctypes.c_int64),
      ('group_offsets', ctypes.c_void_p),
      ('tuning', ctypes.c_int32),
      ('a_k_order', ctypes.c_int32),
      ('k_split', ctypes.c_int32),
      ('k_split_workspace', ctypes.c_void_p), ('k_split_workspace_bytes', ctypes.c_int64),
      ('b_layout', ctypes.c_int32),
      ('accumulate', ctypes.c_int32),
  ]


class GroupedGemmPlan(ctypes.Structure):
  _fields_ = [
      ('m', ctypes.c_int64), ('n', ctypes.c_int64), ('k', ctypes.c_int64), ('group', ctypes.c_int64),
      ('lda', ctypes.c_int64), ('ldb', ctypes.c_int64), ('ldc', ctypes.c_int64),
      ('a_dtype', ctypes.c_int32), ('b_dtype', ctypes.c_int32), ('out_dtype', ctypes.c_int32),
      ('row_scale_dtype', ctypes.c_int32), ('col_scale_dtype', ctypes.c_int32),
      ('a_k_order', ctypes.c_int32), ('row_scale_by_row', ctypes.c_int32), ('tuning', ctypes.c_int32),
  ]


class DecodePlan(ctypes.Structure):
  _fields_ = [
      ('m', ctypes.c_int64), ('n', ctypes.c_int64), ('k', ctypes.c_int64),
      ('x_dtype', ctypes.c_int32), ('x_scale_dtype', ctypes.c_int32),
      ('w_scale_dtype', ctypes.c_int32), ('out_dtype', ctypes.c_int32),
      ('quant_bound', ctypes.c_float), ('clip_bound', ctypes.c_float),
      ('w_dtype', ctypes.c_int32), ('tuning', ctypes.c_int32), ('w_layout', ctypes.c_int32),
      ('workspace_zeroed', ctypes.c_int32),
  ]


# name -> (restype, argtypes); every symbol include/aqtx.h declares
_vp = ctypes.c_void_p
class Im2colPlan(ctypes.Structure):
  _fields_ = [
      ('n', ctypes.c_int64), ('c', ctypes.c_int32), ('rank', ctypes.c_int32),
      ('in_size', ctypes.c_int32 * 3), ('kernel', ctypes.c_int32 * 3), ('stride', ctypes.c_int32 * 3),
      ('dilation', ctypes.c_int32 * 3), ('pad_lo', ctypes.c_int32 * 3), ('out_size', ctypes.c_int32 * 3),
  ]


class FpRoundPlan(ctypes.Structure):
  _fields_ = [
      ('count', ctypes.c_int64), ('noise_mod', ctypes.c_int64),
      ('dtype', ctypes.c_int32), ('nexp', ctypes.c_int32), ('nmant', ctypes.c_int32),
      ('has_subnormals', ctypes.c_int32), ('mode', ctypes.c_int32), ('partitionable', ctypes.c_int32),
      ('radix', ctypes.c_int32),
  ]


FP_NEAREST, FP_NOISE_JAX_BITS, FP_NOISE_INDEX = 0, 1, 2

SYMBOLS = {
    'aqtx_im2col_i8': (ctypes.c_int, [ctypes.POINTER(Im2colPlan), _vp, _vp, _vp]),
    'aqtx_conv_i8': (ctypes.c_int, [ctypes.POINTER(Im2colPlan), ctypes.POINTER(GemmPlan), _vp, _vp, _vp, _vp, _vp, _vp]),
    'aqtx_fp_round': (ctypes.c_int, [ctypes.POINTER(FpRoundPlan), _vp, _vp, ctypes.POINTER(ctypes.c_uint32), _vp]),
    'aqtx_quantize': (ctypes.c_int, [ctypes.POINTER(QuantPlan), _vp, _vp, _vp, _vp, _vp,
                                     ctypes.c_size_t, _vp]),
    'aqtx_quantize_workspace_bytes': (ctypes.c_size_t, [ctypes.POINTER(QuantPlan)]),
    'aqtx_quantize_other_axis_parts': (ctypes.c_int64, [ctypes.POINTER(QuantPlan)]),
    'aqtx_dequantize': (ctypes.c_int, [ctypes.POINTER(QuantPlan), _vp, _vp, _vp, _vp]),
    'aqtx_scale_cast': (ctypes.c_int, [ctypes.POINTER(ScalePlan), _vp, _vp, _vp, _vp, _vp]),
    'aqtx_gemm_i8': (ctypes.c_int, [ctypes.POINTER(GemmPlan), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    'aqtx_gemm_i8_k_slices': (ctypes.c_int, [ctypes.POINTER(GemmPlan)]),
    'aqtx_gemm_fp8': (ctypes.c_int, [ctypes.POINTER(GemmPlan), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    'aqtx_gemm_weight_only': (ctypes.c_int, [ctypes.POINTER(GemmPlan), _vp, _vp, _vp, _vp, _vp]),
    'aqtx_decode_i8': (ctypes.c_int, [ctypes.POINTER(DecodePlan), _vp, _vp, _vp, _vp, _vp, _vp,
                                      _vp, ctypes.c_size_t, _vp]),
    'aqtx_decode_workspace_bytes': (ctypes.c_size_t, [ctypes.POINTER(DecodePlan)]),
    'aqtx_decode_exchange_bytes': (ctypes.c_size_t, [ctypes.POINTER(DecodePlan)]),
    'aqtx_tile_weight_bytes': (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int32]),
    'aqtx_tile_weight': (ctypes.c_int, [_vp, _vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, _vp]),
    'aqtx_decode_i8_check': (ctypes.c_int, [_vp, ctypes.c_size_t, _vp]),
    'aqtx_decode_i8_static': (ctypes.c_int, [ctypes.POINTER(DecodePlan), _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    'aqtx_decode_weight_only': (ctypes.c_int, [ctypes.POINTER(DecodePlan), _vp, _vp, _vp, _vp, _vp, ctypes.c_size_t, _vp]),
    'aqtx_decode_weight_only_workspace_bytes': (ctypes.c_size_t, [ctypes.POINTER(DecodePlan)]),
    'aqtx_gemm_i8_grouped': (ctypes.c_int, [ctypes.POINTER(GroupedGemmPlan), _vp, _vp, _vp, _vp, _vp, _vp]),
    'aqtx_pack_i4': (ctypes.c_int, [_vp, _vp, ctypes.c_int64, _vp]),
    'aqtx_sum_tiles': (ctypes.c_int, [_vp, _vp, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, _vp]),
    'aqtx_prng_split_host': (ctypes.c_int, [ctypes.POINTER(ctypes.c_uint32), ctypes.c_int32,
                                            ctypes.c_int32, ctypes.POINTER(ctypes.c_uint32)]),
    'aqtx_prng_split': (ctypes.c_int, [_vp, ctypes.c_int32, ctypes.c_int32, _vp, _vp]),
    'aqtx_random_bits': (ctypes.c_int, [ctypes.POINTER(ctypes.c_uint32), ctypes.c_int64,
                                        ctypes.c_int32, ctypes.c_int32, _vp, _vp]),
    'aqtx_read_probe': (ctypes.c_int, [_vp, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, _vp, _vp,
                                       ctypes.POINTER(ctypes.c_int32), _vp]),
    'aqtx_last_error': (ctypes.c_char_p, []),
    'aqtx_version': (ctypes.c_int, []),
}

_lib = None


class AqtxError(RuntimeError):
  """A non-zero status from the C-ABI; the message is aqtx_last_error()."""


def lib():
  """Loads libaqtx.so once; raises if it has not been built."""
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(
          f'{LIB_PATH} is missing: build it with `python -m aqt_amd.build` '
          '(there is no CPU fallback for the HIP kernels).')
    handle = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SYMBOLS.items():
      fn = getattr(handle, name)
      fn.restype = restype
      fn.argtypes = argtypes
    _lib = handle
  return _lib


def check(status):
  if status != 0:
    raise AqtxError(lib().aqtx_last_error().decode())

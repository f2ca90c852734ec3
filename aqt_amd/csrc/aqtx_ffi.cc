// XLA FFI handlers over the aqtx C-ABI: what a JAX process registers with
// jax.ffi.register_ffi_target(name, jax.ffi.pycapsule(lib.<Symbol>), platform="ROCM") so that
// aqt.jax.v2's DotGeneralRaw.__call__ (aqt/jax/v2/aqt_dot_general.py:757-840), its lax.dot_general
// call (:921-927) and QTensor.quant / dequant (aqt_tensor.py:125-200) run on the HIP kernels.
//
// Built by aqt_amd/build.py into aqt_amd/lib/libaqtx_ffi.so only where the XLA FFI headers
// (xla/ffi/api/ffi.h; they ship inside jaxlib: jax.ffi.include_dir()) are found.  The handlers
// add nothing to the C-ABI: they read shapes and element types off the XLA buffers, fill the POD
// plans of include/aqtx.h and map a non-zero status to an XLA error carrying aqtx_last_error().
//
// Conventions:
//   * every buffer, including scratch, is an XLA buffer: workspaces are declared as extra uint8
//     results sized with aqtx_*_workspace_bytes() by the Python side that builds the ffi_call;
//   * a PRNG key is a uint32[2] operand in device memory (under jit a key is a traced array, not
//     an attribute); the kernels read it there (aqtx_quant_plan::key_device);
//   * scalars of a plan travel as attributes; a handler without noise still takes the key operand
//     (any uint32[2]), so that one handler serves both;
//   * tensors are passed in the layout the kernels read: [batch, rows, cols] row-major for the
//     quantizers, [batch, m, k] and [batch, n, k] (contraction axis contiguous) for the contractions.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <string>

#include "../../include/aqtx.h"
#include "xla/ffi/api/ffi.h"

namespace ffi = xla::ffi;

namespace {

ffi::Error Status(int rc) {
  if (rc == 0) return ffi::Error::Success();
  return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(aqtx_last_error()));
}

ffi::Error Bad(const char* what) { return ffi::Error(ffi::ErrorCode::kInvalidArgument, std::string(what)); }

// XLA element type -> aqtx element type (-1: not one the kernels take)
int Dtype(ffi::DataType t) {
  switch (t) {
    case ffi::DataType::F32: return AQTX_F32;
    case ffi::DataType::BF16: return AQTX_BF16;
    case ffi::DataType::S8: return AQTX_I8;
    case ffi::DataType::S32: return AQTX_I32;
    case ffi::DataType::F8E4M3FN: return AQTX_E4M3;
    case ffi::DataType::F8E5M2: return AQTX_E5M2;
    default: return -1;
  }
}

// ---- aqtx_quantize ------------------------------------------------------------------------------
// x [batch, rows, cols]; q has the same shape ([batch, cols, rows] with transpose_out); scale f32.
// out_dtype is an attribute because jnp.int4 values live in int8 containers on this side.
ffi::Error QuantizeCommon(hipStream_t stream, ffi::AnyBuffer x, const float* prescale, ffi::Buffer<ffi::U32> key,
                          ffi::Result<ffi::AnyBuffer> q, ffi::Result<ffi::Buffer<ffi::F32>> scale,
                          ffi::Result<ffi::Buffer<ffi::U8>> workspace, int32_t compute_dtype, int32_t scale_dtype,
                          int32_t out_dtype, int32_t reduce, int32_t transpose_out, int64_t group, float quant_bound,
                          float clip_bound, int32_t noise, int32_t partitionable, int64_t noise_stride_batch,
                          int64_t noise_stride_row, int64_t noise_stride_col, int64_t noise_total, int32_t out_k_order,
                          int32_t prescale_mode, int64_t prescale_stride_batch) {
  auto dims = x.dimensions();
  if (dims.size() != 3) return Bad("aqtx_quantize: x must be [batch, rows, cols]");
  if (key.element_count() != 2) return Bad("aqtx_quantize: key must be uint32[2]");
  aqtx_quant_plan p{};
  p.in_dtype = Dtype(x.element_type());
  p.compute_dtype = compute_dtype;
  p.scale_dtype = scale_dtype;
  p.out_dtype = out_dtype;
  p.batch = dims[0]; p.rows = dims[1]; p.cols = dims[2];
  p.reduce = reduce;
  p.transpose_out = transpose_out;
  p.group = group;
  p.quant_bound = quant_bound;
  p.clip_bound = clip_bound;
  p.noise = noise;
  p.partitionable = partitionable;
  p.noise_stride_batch = noise_stride_batch;
  p.noise_stride_row = noise_stride_row;
  p.noise_stride_col = noise_stride_col;
  p.noise_total = noise_total;
  p.out_k_order = out_k_order;
  p.prescale = prescale_mode;
  p.prescale_stride_batch = prescale_stride_batch;
  p.key_device = noise != AQTX_NOISE_NONE ? key.typed_data() : nullptr;
  return Status(aqtx_quantize(&p, x.untyped_data(), prescale, q->untyped_data(), scale->typed_data(),
                              workspace->typed_data(), workspace->size_bytes(), stream));
}

ffi::Error QuantizeImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::U32> key, ffi::Result<ffi::AnyBuffer> q,
                        ffi::Result<ffi::Buffer<ffi::F32>> scale, ffi::Result<ffi::Buffer<ffi::U8>> workspace,
                        int32_t compute_dtype, int32_t scale_dtype, int32_t out_dtype, int32_t reduce,
                        int32_t transpose_out, int64_t group, float quant_bound, float clip_bound, int32_t noise,
                        int32_t partitionable, int64_t noise_stride_batch, int64_t noise_stride_row,
                        int64_t noise_stride_col, int64_t noise_total, int32_t out_k_order) {
  return QuantizeCommon(stream, x, nullptr, key, q, scale, workspace, compute_dtype, scale_dtype, out_dtype, reduce,
                        transpose_out, group, quant_bound, clip_bound, noise, partitionable, noise_stride_batch,
                        noise_stride_row, noise_stride_col, noise_total, out_k_order, AQTX_PRESCALE_NONE, 0);
}

// The gradient side of a backward contraction: x := x * cast(prescale) first
// (_maybe_use_fwd_quant, aqt/jax/v2/aqt_dot_general.py:714-720).
ffi::Error QuantizePrescaledImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::F32> prescale,
                                 ffi::Buffer<ffi::U32> key, ffi::Result<ffi::AnyBuffer> q,
                                 ffi::Result<ffi::Buffer<ffi::F32>> scale, ffi::Result<ffi::Buffer<ffi::U8>> workspace,
                                 int32_t compute_dtype, int32_t scale_dtype, int32_t out_dtype, int32_t reduce,
                                 int32_t transpose_out, int64_t group, float quant_bound, float clip_bound,
                                 int32_t noise, int32_t partitionable, int64_t noise_stride_batch,
                                 int64_t noise_stride_row, int64_t noise_stride_col, int64_t noise_total,
                                 int32_t out_k_order, int32_t prescale_mode, int64_t prescale_stride_batch) {
  return QuantizeCommon(stream, x, prescale.typed_data(), key, q, scale, workspace, compute_dtype, scale_dtype,
                        out_dtype, reduce, transpose_out, group, quant_bound, clip_bound, noise, partitionable,
                        noise_stride_batch, noise_stride_row, noise_stride_col, noise_total, out_k_order,
                        prescale_mode, prescale_stride_batch);
}

// ---- aqtx_dequantize ----------------------------------------------------------------------------
ffi::Error DequantizeImpl(hipStream_t stream, ffi::AnyBuffer q, ffi::Buffer<ffi::F32> scale,
                          ffi::Result<ffi::AnyBuffer> out, int32_t q_dtype, int32_t scale_dtype, int32_t reduce,
                          int64_t group, int32_t transposed) {
  auto dims = out->dimensions();
  if (dims.size() != 3) return Bad("aqtx_dequantize: out must be [batch, rows, cols]");
  aqtx_quant_plan p{};
  p.in_dtype = p.compute_dtype = Dtype(out->element_type());
  p.scale_dtype = scale_dtype;
  p.out_dtype = q_dtype;
  p.batch = dims[0]; p.rows = dims[1]; p.cols = dims[2];
  p.reduce = reduce;
  p.group = group;
  p.transpose_out = transposed;
  p.quant_bound = p.clip_bound = 1.0f;
  return Status(aqtx_dequantize(&p, q.untyped_data(), scale.typed_data(), out->untyped_data(), stream));
}

// ---- aqtx_scale_cast ----------------------------------------------------------------------------
// x [batch, rows, cols] -> out of the same shape; f0 / f1 f32 factor vectors (a one-element dummy for a factor
// the plan does not use).  in_dtype is an attribute for the same reason as out_dtype above.
ffi::Error ScaleCastImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::Buffer<ffi::F32> f0, ffi::Buffer<ffi::F32> f1,
                         ffi::Result<ffi::AnyBuffer> out, int32_t in_dtype, int32_t factors, int32_t factor0_axis,
                         int32_t factor0_dtype, int32_t factor0_recast, int64_t factor0_stride_b,
                         int32_t factor1_axis, int32_t factor1_dtype, int32_t factor1_recast,
                         int64_t factor1_stride_b, int32_t factor0_reciprocal, int32_t factor1_reciprocal,
                         float finish_clip, int32_t finish_round) {
  auto dims = out->dimensions();
  if (dims.size() != 3) return Bad("aqtx_scale_cast: out must be [batch, rows, cols]");
  aqtx_scale_plan p{};
  p.in_dtype = in_dtype;
  p.out_dtype = Dtype(out->element_type());
  p.batch = dims[0]; p.rows = dims[1]; p.cols = dims[2];
  p.factors = factors;
  p.factor_axis[0] = factor0_axis; p.factor_dtype[0] = factor0_dtype;
  p.factor_recast[0] = factor0_recast; p.factor_stride_b[0] = factor0_stride_b;
  p.factor_axis[1] = factor1_axis; p.factor_dtype[1] = factor1_dtype;
  p.factor_recast[1] = factor1_recast; p.factor_stride_b[1] = factor1_stride_b;
  p.factor_reciprocal[0] = factor0_reciprocal; p.factor_reciprocal[1] = factor1_reciprocal;
  p.finish_clip = finish_clip; p.finish_round = finish_round;
  return Status(aqtx_scale_cast(&p, x.untyped_data(), factors > 0 ? f0.typed_data() : nullptr,
                                factors > 1 ? f1.typed_data() : nullptr, out->untyped_data(), stream));
}

// ---- aqtx_gemm_i8 / aqtx_gemm_fp8 ---------------------------------------------------------------
// a [batch, m, k], b [batch, n, k] -> c [batch, m, n]; scales f32 [batch, m] / [batch, n].
int FillGemmPlan(aqtx_gemm_plan* p, const ffi::AnyBuffer& a, const ffi::AnyBuffer& b, ffi::DataType c_type,
                 int32_t a_dtype, int32_t b_dtype, int32_t dequant_dtype, int32_t row_scale_dtype,
                 int32_t col_scale_dtype, int32_t scale_order) {
  auto ad = a.dimensions(), bd = b.dimensions();
  const bool b_packed = b_dtype == AQTX_I4P;  // b is then uint8 [batch, n, k / 2]
  if (ad.size() != 3 || bd.size() != 3 || ad[0] != bd[0] || ad[2] != (b_packed ? 2 * bd[2] : bd[2])) return 1;
  p->batch = ad[0]; p->m = ad[1]; p->n = bd[1]; p->k = ad[2];
  p->lda = p->k; p->ldb = bd[2]; p->ldc = p->n;
  p->stride_a = p->m * p->k; p->stride_b = p->n * bd[2]; p->stride_c = p->m * p->n;
  p->a_dtype = a_dtype; p->b_dtype = b_dtype;
  p->out_dtype = Dtype(c_type);
  p->dequant_dtype = dequant_dtype;
  p->row_scale_dtype = row_scale_dtype; p->col_scale_dtype = col_scale_dtype;
  p->scale_order = scale_order;
  p->row_scale_stride_b = p->m; p->col_scale_stride_b = p->n;
  return 0;
}

// int8 (or int4-in-int8, or b packed int4 as uint8 [batch, n, k / 2]: a_dtype / b_dtype attributes) operands,
// dequantisation fused.  workspace: uint8 [aqtx_gemm_i8_k_slices(plan) * batch * m * n * 4] when that count is
// above 1 (few output tiles and a long k: slices of k leave partial sums there), else any small buffer.
ffi::Error GemmI8Impl(hipStream_t stream, ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::Buffer<ffi::F32> row_scale,
                      ffi::Buffer<ffi::F32> col_scale, ffi::Result<ffi::AnyBuffer> c,
                      ffi::Result<ffi::Buffer<ffi::U8>> workspace, int32_t a_dtype, int32_t b_dtype,
                      int32_t dequant_dtype, int32_t row_scale_dtype, int32_t col_scale_dtype, int32_t scale_order,
                      int32_t a_k_order) {
  aqtx_gemm_plan p{};
  if (FillGemmPlan(&p, a, b, c->element_type(), a_dtype, b_dtype, dequant_dtype, row_scale_dtype, col_scale_dtype,
                   scale_order))
    return Bad("aqtx_gemm_i8: operands must be [batch, m, k] and [batch, n, k]");
  p.a_k_order = a_k_order;
  p.k_split_workspace = workspace->typed_data();  // too small for the slices: the library takes none
  p.k_split_workspace_bytes = (int64_t)workspace->size_bytes();
  return Status(aqtx_gemm_i8(&p, a.untyped_data(), b.untyped_data(), row_scale.typed_data(), col_scale.typed_data(),
                             c->untyped_data(), nullptr, stream));
}

// Raw int32 accumulators (lax.dot_general with preferred_element_type=int32, no scales).
ffi::Error GemmI8RawImpl(hipStream_t stream, ffi::AnyBuffer a, ffi::AnyBuffer b,
                         ffi::Result<ffi::Buffer<ffi::S32>> c) {
  aqtx_gemm_plan p{};
  if (FillGemmPlan(&p, a, b, ffi::DataType::S32, AQTX_I8, AQTX_I8, AQTX_F32, AQTX_F32, AQTX_F32,
                   AQTX_SCALE_ROW_THEN_COL))
    return Bad("aqtx_gemm_i8: operands must be [batch, m, k] and [batch, n, k]");
  return Status(aqtx_gemm_i8(&p, a.untyped_data(), b.untyped_data(), nullptr, nullptr, c->typed_data(), nullptr,
                             stream));
}

// fp8 operands: e4m3fn / e5m2 per operand from the buffers' element types.
ffi::Error GemmFp8Impl(hipStream_t stream, ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::Buffer<ffi::F32> row_scale,
                       ffi::Buffer<ffi::F32> col_scale, ffi::Result<ffi::AnyBuffer> c, int32_t dequant_dtype,
                       int32_t row_scale_dtype, int32_t col_scale_dtype, int32_t scale_order, int32_t accumulate) {
  aqtx_gemm_plan p{};
  if (FillGemmPlan(&p, a, b, c->element_type(), Dtype(a.element_type()), Dtype(b.element_type()), dequant_dtype,
                   row_scale_dtype, col_scale_dtype, scale_order))
    return Bad("aqtx_gemm_fp8: operands must be [batch, m, k] and [batch, n, k]");
  p.accumulate = accumulate;
  return Status(aqtx_gemm_fp8(&p, a.untyped_data(), b.untyped_data(), row_scale.typed_data(), col_scale.typed_data(),
                              c->untyped_data(), nullptr, stream));
}

// ---- aqtx_gemm_i8_grouped -----------------------------------------------------------------------
// a int8 [m, k]; b int8 [n, k] or packed int4 uint8 [n, k/2]; scales f32 [k/group, m] (or [m, k/group] with
// row_scale_by_row), [k/group, n].
ffi::Error GemmI8GroupedImpl(hipStream_t stream, ffi::AnyBuffer a, ffi::AnyBuffer b, ffi::Buffer<ffi::F32> row_scale,
                             ffi::Buffer<ffi::F32> col_scale, ffi::Result<ffi::AnyBuffer> c, int64_t group,
                             int32_t a_dtype, int32_t b_dtype, int32_t row_scale_dtype, int32_t col_scale_dtype,
                             int32_t a_k_order, int32_t row_scale_by_row) {
  auto ad = a.dimensions(), bd = b.dimensions();
  if (ad.size() != 2 || bd.size() != 2) return Bad("aqtx_gemm_i8_grouped: operands must be [m, k] and [n, k]");
  aqtx_grouped_gemm_plan p{};
  p.m = ad[0]; p.k = ad[1]; p.n = bd[0];
  p.group = group;
  p.lda = ad[1]; p.ldb = bd[1]; p.ldc = p.n;  // ldb in bytes for packed int4 = its uint8 row length
  p.a_dtype = a_dtype; p.b_dtype = b_dtype;
  p.out_dtype = Dtype(c->element_type());
  p.row_scale_dtype = row_scale_dtype; p.col_scale_dtype = col_scale_dtype;
  p.a_k_order = a_k_order; p.row_scale_by_row = row_scale_by_row;
  return Status(aqtx_gemm_i8_grouped(&p, a.untyped_data(), b.untyped_data(), row_scale.typed_data(),
                                     col_scale.typed_data(), c->untyped_data(), stream));
}

// ---- aqtx_decode_i8 -----------------------------------------------------------------------------
// x [m, k] bf16/f32, w int8 [n, k] (uint8 [n, k/2] when w_dtype = AQTX_I4P; the flat output of
// aqtx_tile_weight when w_layout = AQTX_W_FRAGMENTS), w_scale f32 [n]
// -> out [m, n], x_scale f32 [m], xq int8 [m, k], workspace uint8[aqtx_decode_workspace_bytes].
ffi::Error DecodeI8Impl(hipStream_t stream, ffi::AnyBuffer x, ffi::AnyBuffer w, ffi::Buffer<ffi::F32> w_scale,
                        ffi::Result<ffi::AnyBuffer> out, ffi::Result<ffi::Buffer<ffi::F32>> x_scale,
                        ffi::Result<ffi::Buffer<ffi::S8>> xq, ffi::Result<ffi::Buffer<ffi::U8>> workspace,
                        float quant_bound, float clip_bound, int32_t x_scale_dtype, int32_t w_scale_dtype,
                        int32_t w_dtype, int32_t w_layout) {
  auto xd = x.dimensions();
  if (xd.size() != 2) return Bad("aqtx_decode_i8: x must be [m, k]");
  aqtx_decode_plan p{};
  p.m = xd[0]; p.k = xd[1];
  p.n = (int64_t)w_scale.element_count();  // a fragment-ordered weight is a flat buffer: n = number of scales
  p.w_layout = w_layout;
  p.x_dtype = Dtype(x.element_type());
  p.x_scale_dtype = x_scale_dtype;
  p.w_scale_dtype = w_scale_dtype;
  p.out_dtype = Dtype(out->element_type());
  p.quant_bound = quant_bound;
  p.clip_bound = clip_bound;
  p.w_dtype = w_dtype;
  return Status(aqtx_decode_i8(&p, x.untyped_data(), w.untyped_data(), w_scale.typed_data(), xq->typed_data(),
                               x_scale->typed_data(), out->untyped_data(), workspace->typed_data(),
                               workspace->size_bytes(), stream));
}

// ---- aqtx_sum_tiles -----------------------------------------------------------------------------
// x [tiles, ...] -> out [...]: the sum over the tile-count axis of tiled_dot_general / LocalAqt.
ffi::Error SumTilesImpl(hipStream_t stream, ffi::AnyBuffer x, ffi::Result<ffi::AnyBuffer> out) {
  auto dims = x.dimensions();
  if (dims.size() < 1) return Bad("aqtx_sum_tiles: x needs a leading tile axis");
  const int64_t tiles = dims[0];
  const int64_t count = tiles == 0 ? 0 : (int64_t)x.element_count() / tiles;
  return Status(aqtx_sum_tiles(x.untyped_data(), out->untyped_data(), tiles, count, Dtype(x.element_type()), stream));
}

}  // namespace

#define AQTX_QUANT_ATTRS()                                                                              \
  .Attr<int32_t>("compute_dtype").Attr<int32_t>("scale_dtype").Attr<int32_t>("out_dtype")              \
  .Attr<int32_t>("reduce").Attr<int32_t>("transpose_out").Attr<int64_t>("group")                       \
  .Attr<float>("quant_bound").Attr<float>("clip_bound").Attr<int32_t>("noise")                         \
  .Attr<int32_t>("partitionable").Attr<int64_t>("noise_stride_batch").Attr<int64_t>("noise_stride_row") \
  .Attr<int64_t>("noise_stride_col").Attr<int64_t>("noise_total").Attr<int32_t>("out_k_order")

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxQuantize, QuantizeImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()           // x
        .Arg<ffi::Buffer<ffi::U32>>()    // key, uint32[2]
        .Ret<ffi::AnyBuffer>()           // q
        .Ret<ffi::Buffer<ffi::F32>>()    // scale
        .Ret<ffi::Buffer<ffi::U8>>()     // workspace
        AQTX_QUANT_ATTRS());

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxQuantizePrescaled, QuantizePrescaledImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()           // x
        .Arg<ffi::Buffer<ffi::F32>>()    // prescale
        .Arg<ffi::Buffer<ffi::U32>>()    // key
        .Ret<ffi::AnyBuffer>()
        .Ret<ffi::Buffer<ffi::F32>>()
        .Ret<ffi::Buffer<ffi::U8>>()
        AQTX_QUANT_ATTRS()
        .Attr<int32_t>("prescale").Attr<int64_t>("prescale_stride_batch"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxDequantize, DequantizeImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Ret<ffi::AnyBuffer>()
        .Attr<int32_t>("q_dtype").Attr<int32_t>("scale_dtype").Attr<int32_t>("reduce")
        .Attr<int64_t>("group").Attr<int32_t>("transposed"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxScaleCast, ScaleCastImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Ret<ffi::AnyBuffer>()
        .Attr<int32_t>("in_dtype").Attr<int32_t>("factors")
        .Attr<int32_t>("factor0_axis").Attr<int32_t>("factor0_dtype").Attr<int32_t>("factor0_recast")
        .Attr<int64_t>("factor0_stride_b")
        .Attr<int32_t>("factor1_axis").Attr<int32_t>("factor1_dtype").Attr<int32_t>("factor1_recast")
        .Attr<int64_t>("factor1_stride_b")
        .Attr<int32_t>("factor0_reciprocal").Attr<int32_t>("factor1_reciprocal")
        .Attr<float>("finish_clip").Attr<int32_t>("finish_round"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxGemmI8, GemmI8Impl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()           // a [batch, m, k]
        .Arg<ffi::AnyBuffer>()           // b [batch, n, k]
        .Arg<ffi::Buffer<ffi::F32>>()    // row scale
        .Arg<ffi::Buffer<ffi::F32>>()    // col scale
        .Ret<ffi::AnyBuffer>()           // c
        .Ret<ffi::Buffer<ffi::U8>>()     // workspace
        .Attr<int32_t>("a_dtype").Attr<int32_t>("b_dtype").Attr<int32_t>("dequant_dtype")
        .Attr<int32_t>("row_scale_dtype").Attr<int32_t>("col_scale_dtype").Attr<int32_t>("scale_order")
        .Attr<int32_t>("a_k_order"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxGemmI8Raw, GemmI8RawImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Ret<ffi::Buffer<ffi::S32>>());

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxGemmFp8, GemmFp8Impl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Ret<ffi::AnyBuffer>()
        .Attr<int32_t>("dequant_dtype").Attr<int32_t>("row_scale_dtype").Attr<int32_t>("col_scale_dtype")
        .Attr<int32_t>("scale_order").Attr<int32_t>("accumulate"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxGemmI8Grouped, GemmI8GroupedImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::AnyBuffer>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Arg<ffi::Buffer<ffi::F32>>()
        .Ret<ffi::AnyBuffer>()
        .Attr<int64_t>("group").Attr<int32_t>("a_dtype").Attr<int32_t>("b_dtype")
        .Attr<int32_t>("row_scale_dtype").Attr<int32_t>("col_scale_dtype")
        .Attr<int32_t>("a_k_order").Attr<int32_t>("row_scale_by_row"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxDecodeI8, DecodeI8Impl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()           // x
        .Arg<ffi::AnyBuffer>()           // w
        .Arg<ffi::Buffer<ffi::F32>>()    // w scale
        .Ret<ffi::AnyBuffer>()           // out
        .Ret<ffi::Buffer<ffi::F32>>()    // x scale
        .Ret<ffi::Buffer<ffi::S8>>()     // xq
        .Ret<ffi::Buffer<ffi::U8>>()     // workspace
        .Attr<float>("quant_bound").Attr<float>("clip_bound").Attr<int32_t>("x_scale_dtype")
        .Attr<int32_t>("w_scale_dtype").Attr<int32_t>("w_dtype").Attr<int32_t>("w_layout"));

XLA_FFI_DEFINE_HANDLER_SYMBOL(
    AqtxSumTiles, SumTilesImpl,
    ffi::Ffi::Bind()
        .Ctx<ffi::PlatformStream<hipStream_t>>()
        .Arg<ffi::AnyBuffer>()
        .Ret<ffi::AnyBuffer>());

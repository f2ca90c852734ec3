/*
 * aqtx -- C-ABI of the MI355X (gfx950) kernels behind the aqt.jax.v2 quantized
 * dot_general path.
 *
 * Conventions (all entry points):
 *   - plain pointers and sizes only; every pointer is a DEVICE pointer unless
 *     its name ends in `_host`;
 *   - the caller owns every buffer (inputs, outputs, workspace); the library
 *     allocates nothing, frees nothing and never synchronises;
 *   - `stream` is a hipStream_t passed as void*; all work is enqueued on it;
 *   - the return value is 0 on success, non-zero otherwise; the message for
 *     the calling thread's last failure is aqtx_last_error();
 *   - argument validation happens before any GPU call, so every error path can
 *     be exercised on a machine without a GPU;
 *   - scales travel as float32 arrays whose values are already rounded to the
 *     scale dtype the plan names (a bf16 scale is a bf16-representable float).
 *
 * The reference (google/aqt) is pure Python on JAX and has no FFI of its own;
 * each entry point below names the reference functions whose XLA-emitted
 * arithmetic it replaces.
 */
#ifndef AQTX_H_
#define AQTX_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define AQTX_VERSION 1

/* element types */
enum {
  AQTX_F32 = 0,
  AQTX_BF16 = 1,
  AQTX_I8 = 2,   /* int8 */
  AQTX_I4 = 3,   /* int4 values in an int8 container (one value per byte) */
  AQTX_E4M3 = 4, /* float8_e4m3fn (OCP) */
  AQTX_E5M2 = 5, /* float8_e5m2 (OCP) */
  AQTX_I32 = 6,
  AQTX_I4P = 7   /* int4 packed two per byte, low nibble = even index */
};

/* which axis of the [batch, rows, cols] view shares one scale */
enum {
  AQTX_REDUCE_COLS = 0, /* one scale per (batch,row[,group])  -> scale[batch][rows][cols/group] */
  AQTX_REDUCE_ROWS = 1, /* one scale per (batch[,group],col)  -> scale[batch][rows/group][cols] */
  AQTX_REDUCE_ALL = 2,  /* one scale per batch entry          -> scale[batch]                   */
  AQTX_REDUCE_ALL_BATCH = 3 /* one scale for the whole tensor  -> scale[1]                       */
};

/* noise added before rounding */
enum {
  AQTX_NOISE_NONE = 0,
  AQTX_NOISE_JAX_UNIFORM = 1,     /* stochastic_rounding.py:36-46  */
  AQTX_NOISE_CUSTOM1 = 2,         /* stochastic_rounding.py:50-78  */
  AQTX_NOISE_FP8_MANTISSA = 3     /* numerics/fp8_numerics.py:36-64 */
};

enum { AQTX_PRESCALE_NONE = 0, AQTX_PRESCALE_PER_ROW = 1, AQTX_PRESCALE_PER_COL = 2 };

/* Order of the bytes of every aligned group of 8 along the contraction (contiguous) axis of a
 * quantized int8 operand.  EVEN_ODD8 stores elements 0,2,4,6,1,3,5,7 of the group: the order in
 * which aqtx_gemm_i8_grouped gets the values of a packed int4 operand out of its nibbles without
 * interleaving them again, so the other operand is written that way by the quantizer. */
enum { AQTX_K_NATURAL = 0, AQTX_K_EVEN_ODD8 = 1 };

/*
 * Plan of one calibrate+quantize pass over a contiguous tensor viewed as
 * [batch, rows, cols] (row-major).
 */
typedef struct aqtx_quant_plan {
  int32_t in_dtype;      /* AQTX_F32 | AQTX_BF16 | AQTX_I8 (int8 values read as floats) */
  int32_t compute_dtype; /* AQTX_F32 | AQTX_BF16: the dtype the reference holds x in   */
  int32_t scale_dtype;   /* AQTX_F32 | AQTX_BF16: Calibration.dtype or compute_dtype    */
  int32_t out_dtype;     /* AQTX_I8 | AQTX_I4 | AQTX_E4M3 | AQTX_E5M2                  */
  int64_t batch, rows, cols;
  int32_t reduce;        /* AQTX_REDUCE_*                                               */
  int32_t transpose_out; /* 1: write q as [batch, cols, rows]                           */
  int64_t group;         /* subchannel size along the reduced axis; 0 = whole axis      */
  float quant_bound;     /* AqtNumerics.get_quant_bound(): 127.5, 7.5, 448, 57344       */
  float clip_bound;      /* forward clip bound: 127, 7, 448, 57344                      */
  int32_t noise;         /* AQTX_NOISE_*                                                */
  int32_t partitionable; /* jax_threefry_partitionable                                  */
  uint32_t key[2];       /* raw threefry key data                                       */
  /* counter of element (b,r,c) in the noise tensor = b*nb + r*nr + c*nc;
     noise_total = number of elements of the noise tensor */
  int64_t noise_stride_batch, noise_stride_row, noise_stride_col, noise_total;
  int32_t prescale;      /* AQTX_PRESCALE_*: x := round(x * cast(v)) first              */
  int32_t scale_given;   /* 1: `scale` is an input (calibration skipped)                */
  int64_t prescale_stride_batch; /* prescale vector of batch b starts at b*this (0 = shared)  */
  void* scale_typed;     /* optional out: the computed scales once more as scale_dtype elements
                            (written for AQTX_BF16 only; NULL or F32: `scale` is all there is)   */
  int32_t workspace_zeroed; /* 1: the caller keeps one workspace across calls on one stream, passes its
                            whole size as workspace_bytes, and its first half is zero on entry;
                            aqtx_quantize returns it zeroed and skips its own clearing launch      */
  const uint32_t* key_device; /* optional DEVICE pointer to the two key words; when not NULL the kernels
                            read the key there and `key` above is ignored (a key that is a traced
                            array under XLA, or one updated on the device between HIP graph replays) */
  int32_t out_k_order;   /* AQTX_K_*: byte order of q along cols; EVEN_ODD8 needs AQTX_REDUCE_COLS, an
                            int8 / int4 out_dtype, no transpose_out, cols and group multiples of 8 */
  /* The backward pass quantizes the int8 values a forward quantizer wrote once more, with scales along the other
     axis (_maybe_use_fwd_quant, aqt/jax/v2/aqt_dot_general.py:675-729), and would read them twice for it (abs-max,
     then quantize).  A forward plan can leave what that abs-max needs behind instead:
     other_axis_absmax: optional out, uint8 [parts][len], parts = aqtx_quantize_other_axis_parts(plan) (0: this plan
     cannot write them), len = the length of the axis this plan reduces over (cols for AQTX_REDUCE_COLS, rows for
     AQTX_REDUCE_ROWS): entry [p][i] = the largest |q| among part p of the values that share position i.
     absmax_partials / absmax_parts: optional in, such an array for THIS plan's input (in_dtype AQTX_I8,
     AQTX_REDUCE_ROWS over whole columns, cols a multiple of 16, batch 1, no prescale, no given scale; [parts][cols],
     16-byte aligned): the abs-max pass
     is skipped and the scales come from the maxima over the parts.  Same results either way. */
  void* other_axis_absmax;
  const void* absmax_partials;
  int64_t absmax_parts;
} aqtx_quant_plan;

/*
 * aqtx_quantize: abs-max calibration + quantization, one launch sequence.
 * Replaces, for one operand: AbsMaxCalibration.get_scale_and_bias_and_sparsity
 * (aqt/jax/v2/calibration.py:117-157), QTensor.quant (aqt_tensor.py:125-159),
 * IntSymmetric.vjp_fwd (numerics/int_numerics.py:81-111), Fp8Numerics.vjp_fwd
 * (numerics/fp8_numerics.py:88-123), the noise functions
 * (stochastic_rounding.py:36-78) and the gradient pre-scaling of
 * _maybe_use_fwd_quant (aqt_dot_general.py:714-720).
 *   x         in  : [batch, rows, cols] of in_dtype
 *   prescale  in  : float32 [rows] or [cols] per batch entry (NULL when plan->prescale == NONE)
 *   q         out : int8 / fp8 bytes, [batch, rows, cols] or transposed
 *   scale     out : float32, layout per plan->reduce (input when scale_given)
 *   workspace     : aqtx_quantize_workspace_bytes(plan) bytes of scratch
 */
int aqtx_quantize(const aqtx_quant_plan* plan, const void* x, const float* prescale,
                  void* q, float* scale, void* workspace, size_t workspace_bytes,
                  void* stream);

/* Scratch bytes aqtx_quantize needs for `plan` (0 for single-pass plans). */
size_t aqtx_quantize_workspace_bytes(const aqtx_quant_plan* plan);

/* Rows of the plan->other_axis_absmax array this plan would write (0: it cannot; leave the pointer NULL). */
int64_t aqtx_quantize_other_axis_parts(const aqtx_quant_plan* plan);

/*
 * aqtx_dequantize: out = cast(q) * scale for a quantized tensor with one scale.
 * Replaces QTensor.dequant (aqt/jax/v2/aqt_tensor.py:161-200) for a tensor
 * that has not gone through a contraction (fake-quant, checkpoint inspection).
 * The plan describes q the way aqtx_quantize wrote it: in_dtype is the
 * dequantized dtype to produce (AQTX_F32 | AQTX_BF16), out_dtype the storage
 * type of q (AQTX_I8 | AQTX_I4 | AQTX_E4M3 | AQTX_E5M2), reduce/group the scale
 * layout, transpose_out whether q is stored [batch, cols, rows].  The result is
 * [batch, rows, cols] of in_dtype.
 */
int aqtx_dequantize(const aqtx_quant_plan* plan, const void* q, const float* scale, void* out,
                    void* stream);

/*
 * Plan of aqtx_scale_cast: one elementwise pass that turns a quantized (or float) tensor into the
 * operand of a FLOAT contraction, or scales the result of one.  x is [batch, rows, cols], row-major;
 * the result has the same shape in out_dtype:
 *     v = cast(x[b, r, c]) rounded to out_dtype
 *     for each factor i < factors, in order:
 *        if factor_recast[i]: v is rounded to out_dtype (and is held in out_dtype from here on)
 *        f = f_i[...], or with factor_reciprocal[i] its reciprocal in factor_dtype[i], 1 where that is infinite
 *            (the reciprocal of QTensor.quant, aqt_tensor.py:151-155)
 *        v = v * f         in the promoted dtype of v and factor_dtype[i] (bf16 x bf16 rounds to bf16;
 *                          anything with a float32 side is a float32 product and v stays float32)
 *     v is rounded to out_dtype; then, in out_dtype:
 *        finish_clip > 0:  v = clip(v, -finish_clip, finish_clip)
 *        finish_round 1:   v = round half to even;  2: v = floor(v) + 0.5
 *     out[b, r, c] = v
 * A factor has one value per (batch, row) (AQTX_FACTOR_ROWS: f_i[b * factor_stride_b[i] + r]) or per
 * (batch, col) (AQTX_FACTOR_COLS: f_i[b * factor_stride_b[i] + c]); stride 0 shares it between the batch
 * entries.  The values are float32 words holding values of factor_dtype[i].
 */
enum { AQTX_FACTOR_ROWS = 0, AQTX_FACTOR_COLS = 1 };

typedef struct aqtx_scale_plan {
  int32_t in_dtype;           /* AQTX_I8 | AQTX_I4 (container) | AQTX_E4M3 | AQTX_E5M2 | AQTX_BF16 | AQTX_F32 */
  int32_t out_dtype;          /* AQTX_BF16 | AQTX_F32                                              */
  int64_t batch, rows, cols;
  int32_t factors;            /* 0, 1 or 2                                                         */
  int32_t factor_axis[2];     /* AQTX_FACTOR_*                                                     */
  int32_t factor_dtype[2];    /* AQTX_BF16 | AQTX_F32: the dtype the factor's values are held in    */
  int32_t factor_recast[2];   /* 1: v is cast to out_dtype before this factor multiplies           */
  int64_t factor_stride_b[2]; /* batch stride of the factor vector, in elements                    */
  int32_t factor_reciprocal[2]; /* 1: the factor multiplies by its reciprocal (a scale that divides)  */
  float finish_clip;          /* > 0: clip bound applied to the result; 0: none                    */
  int32_t finish_round;       /* 0: none, 1: half to even, 2: floor + 0.5                          */
} aqtx_scale_plan;

/*
 * aqtx_scale_cast replaces, for the configurations whose contraction is a float one:
 * QTensor.dequant of one operand before the contraction (DequantMode.THIS_INPUT, _maybe_dequant,
 * aqt/jax/v2/aqt_dot_general.py:853-866, with aqt_tensor.py:161-200: one factor, the operand's own scale),
 * the multiplication by the OTHER operand's transposed scale (DequantMode.OTHER_INPUT,
 * aqt_dot_general.py:887-903: a second factor with factor_recast = 1, or the only one next to a bare cast),
 * the cast of an integer operand that meets a float one in lax.dot_general (no factor), and QTensor.dequant of
 * the contraction's result by the scales of the operands in DequantMode.OUTPUT (aqt_dot_general.py:929-958
 * with aqt_tensor.py:161-200: x float, one factor per such operand); and, with reciprocal factors and the
 * finishing step, QTensor.quant + IntSymmetric.vjp_fwd for numerics whose results stay in the float dtype
 * and need not be integers (round = False, clip = False, preserve_zero = False: aqt_tensor.py:125-159,
 * numerics/int_numerics.py:81-111, without noise).
 *   x   in  : [batch, rows, cols] of in_dtype
 *   f0, f1  : float32 factor vectors (NULL beyond plan->factors)
 *   out out : [batch, rows, cols] of out_dtype (may not alias x unless the dtypes have the same size)
 */
int aqtx_scale_cast(const aqtx_scale_plan* plan, const void* x, const float* f0, const float* f1,
                    void* out, void* stream);

enum { AQTX_SCALE_ROW_THEN_COL = 0, AQTX_SCALE_COL_THEN_ROW = 1 };

/*
 * Plan of C[b] = dequant(A[b] * B[b]^T): A is [batch, m, k], B is [batch, n, k]
 * (both with the contraction axis contiguous), C is [batch, m, n].
 */
#define AQTX_ACC_FAST 0
#define AQTX_ACC_F32 1

typedef struct aqtx_gemm_plan {
  int64_t batch, m, n, k;
  int64_t lda, ldb, ldc;      /* row strides in elements                                    */
  int64_t stride_a, stride_b, stride_c; /* batch strides in elements                      */
  int32_t a_dtype, b_dtype;   /* AQTX_I8 | AQTX_I4 (container) | AQTX_E4M3 | AQTX_E5M2; b_dtype of aqtx_gemm_i8
                                 also AQTX_I4P: int4 packed two per byte ([n][k/2], low nibble = even k, as
                                 aqtx_pack_i4 writes it; ldb and stride_b in bytes, k a multiple of 32),
                                 unpacked in registers on the way to LDS                     */
  int32_t out_dtype;          /* AQTX_BF16 | AQTX_F32 | AQTX_I32 (raw accumulator, no scales) */
  int32_t dequant_dtype;      /* AQTX_BF16 | AQTX_F32: dtype the accumulator is cast to first */
  int32_t row_scale_dtype;    /* AQTX_BF16 | AQTX_F32: dtype of the values in row_scale      */
  int32_t col_scale_dtype;    /* AQTX_BF16 | AQTX_F32: dtype of the values in col_scale      */
  int32_t scale_order;        /* AQTX_SCALE_*: which scale multiplies first                  */
  int64_t row_scale_stride_b, col_scale_stride_b; /* batch strides of the scale vectors    */
  /* Ragged batches (jax.lax.ragged_dot, aqt/jax/v2/aqt_ragged_dot.py:22-46): optional DEVICE
     pointer to batch+1 ascending int32 row offsets.  Entry b multiplies rows
     [off[b], off[b+1]) of one flat A [m, k] with B[b] into the same rows of one flat C [m, n]
     (row_scale is flat [m] too); stride_a, stride_c and row_scale_stride_b are ignored.  Rows
     outside every group are not written.  NULL: ordinary batches.                          */
  const int32_t* group_offsets;
  int32_t tuning;             /* 0 = the library chooses the launch shape.  Tuning only (results never
                                 depend on it): 4 | 8 = waves per workgroup of the int8 kernel on
                                 256 x 256 tiles, one workgroup per tile; 16 = 8 waves, one workgroup per CU
                                 walking the tiles; 128 = the int8 kernel on 128 x 128 tiles, two workgroups a
                                 CU; 129 | 130 | 131 | 132 = its schedule for launches of at most one
                                 workgroup per CU, on 128 x 128 | 64 x 128 | 64 x 64 | 128 x 256 tiles;
                                 133 | 134 = that schedule on 64 x 64 | 64 x 128 tiles with a deeper ring and
                                 one barrier per two stages                                               */
  int32_t a_k_order;          /* AQTX_K_*: byte order of a along k; EVEN_ODD8 (aqtx_gemm_i8 with b_dtype
                                 AQTX_I4P only) saves the kernel the re-interleaving of the nibbles   */
  int32_t k_split;            /* aqtx_gemm_i8 only.  Tuning only (int32 partial sums add up exactly in any
                                 order): 0 = the library chooses, 1 = one workgroup per output tile walks
                                 all of k, S > 1 = k is cut into (at most) S slices contracted by
                                 workgroups of their own, for shapes with few output tiles and a long k.
                                 Slices write partial sums to k_split_workspace                        */
  void* k_split_workspace;    /* DEVICE scratch for the slices, 16-byte aligned, at least
                                 aqtx_gemm_i8_k_slices(plan) * batch * m * n * 4 bytes; NULL: no slices
                                 unless k_split > 1 asks for them (then an error)                      */
  int64_t k_split_workspace_bytes;
  int32_t b_layout;           /* aqtx_gemm_i8 and aqtx_gemm_weight_only.  AQTX_W_ROWS (0): b is [batch][n][k] rows.
                                 AQTX_W_FRAGMENTS: b is one weight (batch 1; int8, or AQTX_I4P) re-laid by
                                 aqtx_tile_weight, the copy the serving kernels stream; ldb and stride_b are
                                 ignored.  Same results                                                 */
  int32_t accumulate;         /* aqtx_gemm_fp8 only.  AQTX_ACC_FAST (0): the fp8 matrix instruction
                                 (v_mfma_scale_f32_32x32x64_f8f6f4), which aligns the products of every 8 consecutive k
                                 to the largest of them and cuts each off 2^-13 below it before they are summed.
                                 AQTX_ACC_F32: both operands are widened to bf16 (exactly) on their way to the
                                 matrix cores (v_mfma_f32_32x32x16_bf16): sums within the error bound of a float32
                                 summation, at half the matrix-core rate                                */
} aqtx_gemm_plan;

/*
 * aqtx_gemm_i8: int8 x int8 -> int32 MFMA contraction with the dequantisation
 * fused in the epilogue.  Replaces _qtensor_dot_general
 * (aqt/jax/v2/aqt_dot_general.py:843-958, the lax.dot_general call at :921-927
 * with preferred_element_type=int32) followed by QTensor.dequant
 * (aqt_tensor.py:161-200): out = cast(acc) * first_scale * second_scale, each
 * product rounded to the promoted dtype of its two operands (so a bf16 value
 * times a bf16 scale rounds to bf16, and anything times an f32 scale stays
 * f32 from then on), final cast to out_dtype.
 *   row_scale : float32 [batch][m] or NULL (= no scale on that side)
 *   col_scale : float32 [batch][n] or NULL
 *   acc_out   : optional int32 [batch][m][n] copy of the raw accumulators
 */
int aqtx_gemm_i8(const aqtx_gemm_plan* plan, const void* a, const void* b,
                 const float* row_scale, const float* col_scale, void* c,
                 int32_t* acc_out, void* stream);

/*
 * Slices of k aqtx_gemm_i8 takes for `plan` when plan->k_split_workspace is large enough (see
 * plan->k_split); 1 = none, no workspace needed.  No counterpart in the reference (XLA picks its own
 * contraction algorithm).
 */
int aqtx_gemm_i8_k_slices(const aqtx_gemm_plan* plan);

/*
 * aqtx_gemm_weight_only: c[m, n] = bf16(bf16(sum_k a[m, k] * float(b[n, k])) * col_scale[n]) for bf16
 * activations that are NOT quantized and an int8 (or int4 in int8 containers) weight, any m.  Replaces
 * _qtensor_dot_general with an unquantized lhs (aqt/jax/v2/aqt_dot_general.py:843-958: the quantized rhs is
 * promoted to bf16, lax.dot_general contracts in float) followed by QTensor.dequant with the rhs scale
 * (aqt_tensor.py:161-200), without the bf16 copy of the weight: the int8 bytes are widened (exactly) on their
 * way into v_mfma_f32_32x32x16_bf16.  Float32 sums: agrees with the reference's float contraction to summation
 * order, not bit for bit.  Of the plan: batch, m, n, k, lda, ldb (elements), ldc, strides, a_dtype (AQTX_BF16),
 * b_dtype (AQTX_I8 | AQTX_I4), out_dtype = dequant_dtype = AQTX_BF16, col_scale_dtype, col_scale_stride_b are
 * read.  k % 16 == 0, lda % 8 == 0, ldb % 16 == 0, a and b 16-byte aligned.  For m <= 64 aqtx_decode_weight_only
 * streams the weight faster.
 */
int aqtx_gemm_weight_only(const aqtx_gemm_plan* plan, const void* a, const void* b, const float* col_scale,
                          void* c, void* stream);

/*
 * aqtx_gemm_fp8: fp8 x fp8 -> float32 MFMA contraction (a_dtype/b_dtype select
 * e4m3fn or e5m2 per operand), same epilogue as aqtx_gemm_i8.  Replaces the
 * same reference lines with preferred_element_type=float32
 * (aqt_dot_general.py:119-121).  Float sums: the result agrees with the reference's
 * float32 contraction to the summation order and, with plan->accumulate == AQTX_ACC_FAST,
 * to the reduced-precision product alignment of the fp8 matrix instruction;
 * AQTX_ACC_F32 keeps the sums within the error bound of a float32 summation.
 */
int aqtx_gemm_fp8(const aqtx_gemm_plan* plan, const void* a, const void* b,
                  const float* row_scale, const float* col_scale, void* c,
                  float* acc_out, void* stream);

/*
 * Plan of a contraction whose operands carry one scale per `group` consecutive
 * elements of the contraction axis (subchannel / tiled quantization).
 */
typedef struct aqtx_grouped_gemm_plan {
  int64_t m, n, k;
  int64_t group;              /* multiple of 128 that divides k                            */
  int64_t lda, ldb, ldc;      /* row strides in elements (ldb in bytes for AQTX_I4P)        */
  int32_t a_dtype;            /* AQTX_I8 | AQTX_I4                                          */
  int32_t b_dtype;            /* AQTX_I8 | AQTX_I4 | AQTX_I4P (packed, low nibble = even k) */
  int32_t out_dtype;          /* AQTX_BF16 | AQTX_F32: dequant dtype = output dtype         */
  int32_t row_scale_dtype, col_scale_dtype; /* AQTX_BF16 | AQTX_F32                         */
  int32_t a_k_order;          /* AQTX_K_*: byte order of a along k; EVEN_ODD8 needs b_dtype AQTX_I4P */
  int32_t row_scale_by_row;   /* 0: row_scale is [k/group][m]; 1: [m][k/group], as aqtx_quantize
                                 with AQTX_REDUCE_COLS and a group writes it                  */
  int32_t tuning;             /* 0 = the library chooses the kernel.  Tuning only (results never depend on
                                 it): 128 = the tile kernels also for m <= 64 (group 128 otherwise goes to
                                 a kernel with one wave per 16 rows of b and no padding of m)  */
} aqtx_grouped_gemm_plan;

/*
 * aqtx_gemm_i8_grouped: C[m,n] = cast(sum_g dequant_g(sum_{k in g} A[m,k] B[n,k])) with
 * dequant_g = QTensor.dequant with the scales of group g.  Replaces tiled_dot_general
 * (aqt/jax/v2/tiled_dot_general.py:407-543) around a quantizing dot_general for a tiled
 * contraction axis: the inner per-tile contractions (tile-count axis as a batch axis,
 * :430-435), their dequantisation (aqt_tensor.py:161-200, each tile rounded to the dequant
 * dtype) and the sum over tiles (:493, float32 accumulation in tile order), without
 * materialising the per-tile outputs.
 *   a          : int8 [m][lda]
 *   b          : int8 [n][ldb], or packed int4 [n][ldb bytes]
 *   row_scale  : float32 [k/group][m]   (scale of A's row m in group g), or [m][k/group] with row_scale_by_row
 *   col_scale  : float32 [k/group][n]
 *   c          : [m][ldc] of out_dtype
 */
int aqtx_gemm_i8_grouped(const aqtx_grouped_gemm_plan* plan, const void* a, const void* b,
                         const float* row_scale, const float* col_scale, void* c, void* stream);

/*
 * aqtx_pack_i4: `count` int4 values held one per int8 byte -> count/2 bytes, two per byte
 * (low nibble = even index).  The reference stores jnp.int4 arrays (int_numerics.py:109-110);
 * the packed layout is this library's storage format for frozen int4 weights.
 */
int aqtx_pack_i4(const void* src, void* dst, int64_t count, void* stream);

/*
 * aqtx_sum_tiles: out[i] = cast(sum over t of x[t][i]) for x [tiles][count] of
 * bf16 or f32, accumulated in float32 in tile order and rounded once.  Replaces
 * the sum over the tile-count axes of the per-tile (already dequantized) outputs
 * in tiled_dot_general (aqt/jax/v2/tiled_dot_general.py:493).
 */
int aqtx_sum_tiles(const void* x, void* out, int64_t tiles, int64_t count, int32_t dtype,
                   void* stream);

/*
 * aqtx_im2col_i8: the windows of a quantized convolution input x [n][spatial...][c] (int8, one to
 * three spatial axes, features innermost) as rows of out [n * positions][taps * c]: columns in
 * the kernel's row-major tap order with the features innermost, zeros in the padding.  With it
 * lax.conv_general_dilated on the quantized values (aqt/jax/v2/aqt_conv_general.py:95-107, Flax
 * layout) is aqtx_gemm_i8 of out with the kernel reshaped to [features_out][taps * c].
 * out_size[d] must be the number of window positions along axis d, i.e.
 * (pad_lo + in_size + pad_hi - ((kernel - 1) * dilation + 1)) / stride + 1.
 */
typedef struct aqtx_im2col_plan {
  int64_t n;            /* images */
  int32_t c;            /* features */
  int32_t rank;         /* spatial axes, 1..3 */
  int32_t in_size[3], kernel[3], stride[3], dilation[3], pad_lo[3], out_size[3];
} aqtx_im2col_plan;

int aqtx_im2col_i8(const aqtx_im2col_plan* plan, const void* x, void* out, void* stream);

/*
 * aqtx_conv_i8: the same convolution in one launch, the windows read in place instead of gathered:
 * C[images * positions][n] = dequant(windows(x) * B^T), i.e. aqtx_im2col_i8(window, x) followed by
 * aqtx_gemm_i8(plan, ., b, ...) without the [images * positions][taps * c] matrix in between (same bits).
 * Replaces the same reference lines (aqt/jax/v2/aqt_conv_general.py:95-107).  `plan` describes the
 * contraction (batch 1, m = images * positions, n, k = taps * c, ldb, ldc, dtypes, scale order; lda is not
 * read); features must be a multiple of 128 and x smaller than 2 GiB, other inputs take the two calls.
 *   x : int8 [images][spatial...][c];  b : int8 [n][ldb];  row_scale float32 [m], col_scale float32 [n]
 */
int aqtx_conv_i8(const aqtx_im2col_plan* window, const aqtx_gemm_plan* plan, const void* x, const void* b,
                 const float* row_scale, const float* col_scale, void* c, void* stream);

/*
 * aqtx_fp_round: rounds x[count] (bf16 or f32) to an emulated small float with `nexp`
 * exponent bits, `nmant` mantissa bits, smallest exponent 0, with or without subnormals, no
 * NaN/inf codes, and writes the result in the same container dtype.  Replaces
 * fp_numerics.fp_round for radix 2 (aqt/jax/v2/numerics/fp_numerics.py:279-459), which
 * FpNumerics.vjp_fwd calls on the bf16 cast of its input (fp_numerics.py:632-640).
 * With radix = 4 the result is sign(x) * 4^floor(log4(1.6 |x|)) (nearest), or
 * sign(x) * 4^floor(log4(|x| + u * (width of x's bucket))) with u in [0, 1) from 16 random bits
 * (stochastic), zero below 4^-3 and +-64 from 4^3 up.  floor(log4(.)) is taken from the float32
 * exponent (exact), where the reference divides two float32 logarithms: the two can differ only
 * where the argument is a power of 4 to within an ulp, points the reference's own test leaves
 * out (fp_numerics_test.py:364-377).
 *   AQTX_FP_NEAREST        : half a truncated ulp is added to the bit pattern
 *   AQTX_FP_NOISE_JAX_BITS : stochastic rounding with jax.random.bits(key, [count], uint16)
 *   AQTX_FP_NOISE_INDEX    : stochastic rounding with noise = index % noise_mod, the
 *                            reference's equi-spaced test noise along the last axis
 *                            (test_noise_axis, fp_numerics.py:334-340)
 */
enum { AQTX_FP_NEAREST = 0, AQTX_FP_NOISE_JAX_BITS = 1, AQTX_FP_NOISE_INDEX = 2 };

typedef struct aqtx_fp_round_plan {
  int64_t count;
  int64_t noise_mod;      /* AQTX_FP_NOISE_INDEX only: 1..65536 */
  int32_t dtype;          /* AQTX_BF16 | AQTX_F32 */
  int32_t nexp;           /* 0..7 */
  int32_t nmant;          /* below the container's mantissa width (7 / 23) */
  int32_t has_subnormals;
  int32_t mode;
  int32_t partitionable;  /* jax_threefry_partitionable layout of the random bits */
  int32_t radix;          /* 0 or 2: the format described by nexp / nmant / has_subnormals; 4: the
                             reference's RADIX4 format {0, +-4^-3 .. +-4^3} (fp_numerics.py:661-706),
                             bf16 only; nexp, nmant and has_subnormals are then not read */
} aqtx_fp_round_plan;

int aqtx_fp_round(const aqtx_fp_round_plan* plan, const void* x, void* out,
                  const uint32_t key_host[2], void* stream);

/*
 * Plan of the serving contraction out[m, n] = dequant(quant(x)[m, k] * W[n, k]^T)
 * with a pre-quantized weight (QTensor: int8 qvalue + per-output-channel scale)
 * and per-token dynamic int8 quantisation of the activations, m <= 64.
 */
/* layout of the weight aqtx_decode_i8 reads */
enum {
  AQTX_W_ROWS = 0,      /* [n][k] (uint8 [n][k/2] for AQTX_I4P), the contraction axis contiguous               */
  AQTX_W_FRAGMENTS = 1  /* written by aqtx_tile_weight: [ceil(n/16)][ceil(row bytes/64)][1 KiB], each KiB the
                           operand bytes of one MFMA fragment (16 rows x 64 bytes) in lane order, zero padded.
                           One wave load is then one contiguous KiB instead of 16 pieces a row apart: the
                           weight streams 20-25 % faster.  This library's storage format for frozen weights.  */
};

typedef struct aqtx_decode_plan {
  int64_t m, n, k;
  int32_t x_dtype;        /* AQTX_BF16 | AQTX_F32                       */
  int32_t x_scale_dtype;  /* dtype the activation scale is rounded to   */
  int32_t w_scale_dtype;  /* dtype of the weight scale (values in f32)  */
  int32_t out_dtype;      /* AQTX_BF16 | AQTX_F32                       */
  float quant_bound, clip_bound; /* of the activation numerics        */
  int32_t w_dtype;        /* AQTX_I8 | AQTX_I4 (container) | AQTX_I4P (packed: k multiple of 32) */
  int32_t tuning;         /* 0 = the library chooses the launch shape.  Tuning only (results never
                             depend on it): bits 0-7 K ranges per weight tile, bits 8-11 16-row weight
                             blocks per wave (1 | 2 | 4), bits 12-15 K steps in flight per wave (2 | 4 |
                             8 | 15 = 16; capped by the register file),
                             bits 16-19 path: 1 = few tokens take the path of many as well (no kernel in
                             which every workgroup quantizes the activations itself), 2 = that, with
                             the activations quantized by a launch of their own.  Bits 20-23: 1 = the
                             wait of aqtx_decode_i8_check's description expires at once (error-path tests)  */
  int32_t w_layout;       /* AQTX_W_ROWS | AQTX_W_FRAGMENTS */
  int32_t workspace_zeroed; /* 1: the caller keeps one workspace across calls on one stream and its first
                             aqtx_decode_exchange_bytes(plan) bytes were zero before the first call.
                             Every call leaves them zero (the kernels reset the words they use), so
                             later calls may say 1 again and no call has to clear them.  The rest of
                             the scratch lives in the LAST bytes of the workspace: one shared by plans
                             of different shapes must hold the largest exchange size plus the largest
                             (workspace_bytes - exchange_bytes) of those plans.                      */
} aqtx_decode_plan;

/*
 * aqtx_decode_i8: fused activation quantisation + skinny int8 contraction +
 * dequantisation for serving (pre-quantized rhs).  Replaces
 * DotGeneralRaw.__call__ (aqt/jax/v2/aqt_dot_general.py:757-840) called with a
 * full rhs_qt, i.e. quant() of the lhs only (:598-672), the int32 dot and
 * QTensor.dequant; the standalone reference equivalents are
 * pallas/quantizer.py:33-68 and pallas/dot_general.py:57-137.
 *   x        in  : [m, k] activations
 *   w        in  : int8 [n, k] (weight stored with the contraction axis contiguous), or
 *                  uint8 [n, k/2] for AQTX_I4P (aqtx_pack_i4 layout); either of them in fragment
 *                  order (aqtx_tile_weight) when plan->w_layout = AQTX_W_FRAGMENTS
 *   w_scale  in  : float32 [n]
 *   xq       out : optional int8 [m, k] (the quantized activations), may be NULL
 *   x_scale  out : float32 [m]
 *   out      out : [m, n]
 *   workspace    : aqtx_decode_workspace_bytes(plan) bytes, 256-byte aligned, any contents (the
 *                  partial sums of the K ranges and, when xq is NULL, the quantized activations)
 */
int aqtx_decode_i8(const aqtx_decode_plan* plan, const void* x, const void* w,
                   const float* w_scale, void* xq, float* x_scale, void* out,
                   void* workspace, size_t workspace_bytes, void* stream);
size_t aqtx_decode_workspace_bytes(const aqtx_decode_plan* plan);
/* Leading bytes of the workspace that hold the partial-sum exchange and the control words (see workspace_zeroed). */
size_t aqtx_decode_exchange_bytes(const aqtx_decode_plan* plan);
/*
 * aqtx_decode_i8_check: with plan->workspace_zeroed, three to 32 tokens and a weight of 24 MiB or more,
 * aqtx_decode_i8 is one launch in which the first m workgroups quantize a token each while the others already
 * stream their weights and then wait for those tokens behind a bounded loop (0.2 s).  A wait that expires (it never should: the quantizing
 * workgroups are resident first) leaves the call's outputs unwritten and a mark in the workspace; no kernel
 * hangs.  This function reads the mark (it synchronizes the stream: call it where the caller synchronizes anyway,
 * not under graph capture), returns 0 if no wait has expired since the workspace was zeroed or last checked, and
 * otherwise an error after clearing the control words.  No counterpart in the reference.
 */
int aqtx_decode_i8_check(void* workspace, size_t workspace_bytes, void* stream);

/*
 * aqtx_tile_weight: a frozen weight [n][k] (int8, or packed int4 as uint8 [n][k/2]) -> AQTX_W_FRAGMENTS order,
 * aqtx_tile_weight_bytes(n, k, w_dtype) bytes at dst.  Done once per frozen tensor; the reference keeps
 * QTensor.qvalue in logical order (aqt/jax/v2/aqt_tensor.py:55-94), the fragment order is this library's
 * serving format next to it (like the packed int4 form).
 */
size_t aqtx_tile_weight_bytes(int64_t n, int64_t k, int32_t w_dtype);
int aqtx_tile_weight(const void* src, void* dst, int64_t n, int64_t k, int32_t w_dtype, void* stream);

/*
 * aqtx_decode_i8_static: aqtx_decode_i8 without the workspace argument.  It has no counterpart in
 * the reference; it is for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  The partial sums and the
 * fragment-ordered activations live in a 10.6 MB array built into the library's device code (one
 * copy per GPU, held until the process ends); the call makes no allocation, copy, memset or
 * synchronisation.  Limits: n <= 32768 and k <= 32768 (larger plans are rejected with an error;
 * use aqtx_decode_i8).  plan->workspace_zeroed is ignored.  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (different streams or host threads) race; calls on
 * one stream are ordered and safe.  The first call on a GPU looks up the array's device address
 * and must not be made while a stream of that GPU is being captured.
 */
int aqtx_decode_i8_static(const aqtx_decode_plan* plan, const void* x, const void* w,
                          const float* w_scale, void* xq, float* x_scale, void* out, void* stream);

/*
 * aqtx_decode_weight_only: out[m, n] = dequant(x[m, :] . float(w[n, :])) for m <= 64 bf16 activations that are
 * NOT quantized and a frozen int8 / int4 weight with one scale per output channel.  Replaces
 * _qtensor_dot_general with an unquantized lhs (aqt/jax/v2/aqt_dot_general.py:843-958: the quantized rhs is
 * promoted to the lhs dtype, lax.dot_general contracts in float, the rhs scale multiplies the output) followed
 * by QTensor.dequant (aqt_tensor.py:161-200), for a provided rhs QTensor (:614-635).  The weight is streamed
 * once and converted to bf16 in registers; sums are float32, so the result agrees with the reference's float
 * contraction to summation order, not bit for bit.  Of the plan: m, n, k, x_dtype (AQTX_BF16), w_dtype,
 * w_layout, w_scale_dtype, out_dtype and tuning (low three bits 1 / 2 / 4: weight rows per workgroup in
 * sixteens, bits 4-7: slices of k; 0 = the library chooses) are read.  k must be a multiple of 16 (32 for
 * packed int4).
 */
int aqtx_decode_weight_only(const aqtx_decode_plan* plan, const void* x, const void* w, const float* w_scale,
                            void* out, void* workspace, size_t workspace_bytes, void* stream);
/* Scratch bytes with which aqtx_decode_weight_only cuts k into slices for `plan` (more than 16 tokens against a
   weight of few rows; float32 partial sums, added in slice order); 0 = it would not.  The workspace is optional:
   without it (NULL) the call walks all of k per workgroup. */
size_t aqtx_decode_weight_only_workspace_bytes(const aqtx_decode_plan* plan);

/*
 * aqtx_prng_split_host: jax.random.split(key, num) on the host (used by
 * config.set_context, aqt/jax/v2/config.py:61-90).  out_host: uint32[num][2].
 */
int aqtx_prng_split_host(const uint32_t key_host[2], int32_t num, int32_t partitionable,
                         uint32_t* out_host);

/*
 * aqtx_prng_split: the same split of a key held in DEVICE memory, by a kernel: key_device uint32[2],
 * out_device uint32[num][2].  For keys that are traced arrays under XLA or change between replays of a
 * HIP graph (aqtx_quant_plan.key_device reads the results).
 */
int aqtx_prng_split(const uint32_t* key_device, int32_t num, int32_t partitionable, uint32_t* out_device,
                    void* stream);

/*
 * aqtx_random_bits: jax.random.bits(key, [n], uint{bit_width}) on the device,
 * bit_width in {16, 32}; out is uint16[n] or uint32[n].  Exposes the in-kernel
 * generator of aqtx_quantize for tests (stochastic_rounding.py:46,65).
 */
int aqtx_random_bits(const uint32_t key_host[2], int64_t n, int32_t bit_width,
                     int32_t partitionable, void* out, void* stream);

/*
 * aqtx_read_probe: a measurement aid with no counterpart in the reference and no use in the product path.
 * Streams `bytes` (a multiple of 16, below 2 GiB) from src once and does nothing else, so that the serving
 * kernels can be set against what the memory system delivers to a pure reader of the same bytes.  The launch
 * shape is the caller's: `workgroups` of 256 lanes walk chunks of 256 * loads_in_flight * 16 bytes round-robin
 * (0 = one workgroup per chunk), loads_in_flight (2 | 4 | 8 | 16) loads of 16 bytes per lane are in flight, a
 * wave load is one contiguous KiB, cache_policy (0..3) is the cache-policy field of the buffer loads (bit 1 =
 * non-temporal).  out_words: uint32 [65536] DEVICE, one checksum word per workgroup XORed in.  stamps: optional
 * uint64 [2 * workgroups] DEVICE: every workgroup's first and last reading of the constant-rate device clock,
 * whose rate in kHz goes to *wall_clock_khz (optional, HOST): max(last) - min(first) is the span of the launch.
 */
int aqtx_read_probe(const void* src, int64_t bytes, int32_t workgroups, int32_t loads_in_flight,
                    int32_t cache_policy, void* out_words, uint64_t* stamps, int32_t* wall_clock_khz,
                    void* stream);

/* Message of the calling thread's most recent failure ("" if none). */
const char* aqtx_last_error(void);

/* AQTX_VERSION the library was built from. */
int aqtx_version(void);

#ifdef __cplusplus
}
#endif
#endif /* AQTX_H_ */

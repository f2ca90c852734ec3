// int8 x int8 -> int32 contraction on gfx950 MFMA (v_mfma_i32_32x32x32_i8) with the
// dequantisation fused in the epilogue; the kernel lives in gemm_core.h.
#include <atomic>

#include "gemm_core.h"

namespace aqtx {

int validate_gemm_plan(const aqtx_gemm_plan* p, const char* who, bool fp8) {
  AQTX_REQUIRE(p != nullptr, "%s: plan is NULL", who);
  AQTX_REQUIRE(p->batch >= 0 && p->m >= 0 && p->n >= 0 && p->k >= 0, "%s: negative shape", who);
  if (fp8) {
    AQTX_REQUIRE((p->a_dtype == AQTX_E4M3 || p->a_dtype == AQTX_E5M2) &&
                     (p->b_dtype == AQTX_E4M3 || p->b_dtype == AQTX_E5M2),
                 "%s: operands must be e4m3/e5m2 (got %d, %d)", who, p->a_dtype, p->b_dtype);
    AQTX_REQUIRE(p->out_dtype == AQTX_BF16 || p->out_dtype == AQTX_F32,
                 "%s: out_dtype must be bf16 or f32, got %d", who, p->out_dtype);
  } else {
    AQTX_REQUIRE((p->a_dtype == AQTX_I8 || p->a_dtype == AQTX_I4) &&
                     (p->b_dtype == AQTX_I8 || p->b_dtype == AQTX_I4 || p->b_dtype == AQTX_I4P),
                 "%s: operands must be int8 containers, b also packed int4 (got %d, %d)", who, p->a_dtype, p->b_dtype);
    AQTX_REQUIRE(p->out_dtype == AQTX_BF16 || p->out_dtype == AQTX_F32 || p->out_dtype == AQTX_I32,
                 "%s: out_dtype must be bf16, f32 or i32, got %d", who, p->out_dtype);
  }
  AQTX_REQUIRE(p->accumulate == AQTX_ACC_FAST || (fp8 && p->accumulate == AQTX_ACC_F32 && p->group_offsets == nullptr),
               "%s: accumulate must be AQTX_ACC_FAST, or AQTX_ACC_F32 for fp8 operands without ragged batches", who);
  AQTX_REQUIRE(is_float_dtype(p->dequant_dtype), "%s: dequant_dtype must be bf16 or f32", who);
  AQTX_REQUIRE(is_float_dtype(p->row_scale_dtype) && is_float_dtype(p->col_scale_dtype),
               "%s: row_scale_dtype / col_scale_dtype must be bf16 or f32", who);
  AQTX_REQUIRE(p->scale_order == AQTX_SCALE_ROW_THEN_COL || p->scale_order == AQTX_SCALE_COL_THEN_ROW,
               "%s: unknown scale_order %d", who, p->scale_order);
  const bool b_packed = !fp8 && p->b_dtype == AQTX_I4P;
  AQTX_REQUIRE(p->lda >= p->k && (p->b_layout == AQTX_W_FRAGMENTS || p->ldb >= (b_packed ? p->k / 2 : p->k)) && p->ldc >= p->n,
               "%s: leading dimension smaller than the row length", who);
  AQTX_REQUIRE(p->a_k_order == AQTX_K_NATURAL || (p->a_k_order == AQTX_K_EVEN_ODD8 && b_packed),
               "%s: a_k_order must be AQTX_K_NATURAL, or AQTX_K_EVEN_ODD8 with a packed int4 b", who);
  AQTX_REQUIRE(!b_packed || (p->k % 32 == 0 && p->k * (int64_t)(127 * 8 * 16) < (1ll << 31)),
               "%s: a packed int4 b needs k to be a multiple of 32 below 132096, got %lld", who, (long long)p->k);
  AQTX_REQUIRE(p->batch <= 65535 && p->m <= (int64_t)65535 * 256, "%s: shape too large for one launch", who);
  AQTX_REQUIRE(p->b_layout == AQTX_W_ROWS || (p->b_layout == AQTX_W_FRAGMENTS && !fp8 && p->batch <= 1 &&
                                              p->group_offsets == nullptr && p->k > 0 && p->k % (b_packed ? 32 : 16) == 0),
               "%s: b_layout must be AQTX_W_ROWS, or AQTX_W_FRAGMENTS for one int8 / packed int4 weight (batch 1, no "
               "ragged batches, k a multiple of 16 / 32)", who);
  AQTX_REQUIRE(p->b_layout == AQTX_W_ROWS || ((p->n + 15) / 16) * (((b_packed ? p->k / 2 : p->k) + 63) / 64) * 1024 < (1ll << 31),
               "%s: fragment-ordered weight larger than 2 GiB", who);
  return 0;
}

}  // namespace aqtx

namespace aqtx {
// CUs of the current device, asked once per device.
int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}
}  // namespace aqtx

using namespace aqtx;


extern "C" int aqtx_gemm_i8_k_slices(const aqtx_gemm_plan* p) {
  if (p == nullptr || p->k_split < 0 || p->k_split > 64 || p->batch <= 0 || p->m <= 0 || p->n <= 0) return 1;
  const int s = gemm_mid_k_slices(p);
  return s > 1 ? s : 1;
}

extern "C" int aqtx_gemm_i8(const aqtx_gemm_plan* p, const void* a, const void* b,
                            const float* row_scale, const float* col_scale, void* c,
                            int32_t* acc_out, void* stream) {
  clear_error();
  if (int rc = validate_gemm_plan(p, "aqtx_gemm_i8", false)) return rc;
  if (p->batch == 0 || p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "aqtx_gemm_i8: NULL buffer");
  AQTX_REQUIRE(p->out_dtype != AQTX_I32 || (row_scale == nullptr && col_scale == nullptr),
               "aqtx_gemm_i8: raw int32 output takes no scales");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)c % esz) == 0, "aqtx_gemm_i8: output is not element aligned");

  GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  g.a_even_odd8 = p->a_k_order == AQTX_K_EVEN_ODD8;
  const bool b_packed = p->b_dtype == AQTX_I4P;
  g.b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  g.b_steps = (int)(((b_packed ? p->k / 2 : p->k) + 63) / 64);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);

  const bool b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  if (!gemm_vector_path_ok(p, a, b)) {
    AQTX_REQUIRE(!b_packed && !b_frag,
                 "aqtx_gemm_i8: a packed int4 or fragment-ordered b needs 16-byte aligned operands and leading dimensions");
    AQTX_REQUIRE(p->group_offsets == nullptr,
                 "aqtx_gemm_i8: ragged batches need 16-byte aligned operands with k and leading dimensions "
                 "multiple of 16");
    dim3 grid((unsigned)((p->n + 255) / 256), (unsigned)p->m, (unsigned)p->batch);
    AQTX_REQUIRE(p->m <= 65535, "aqtx_gemm_i8: m too large for the unaligned path");
    gemm_simple_kernel<DecI8, DecI8, true><<<grid, 256, 0, st>>>(g);
    AQTX_HIP_CHECK_LAUNCH("gemm_simple_kernel");
    return 0;
  }
  AQTX_REQUIRE(p->lda * (int64_t)BM < (1ll << 31) && p->ldb * (int64_t)BN < (1ll << 31),
               "aqtx_gemm_i8: leading dimension too large for 32-bit tile offsets");
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  const int epi = gemm_epilogue_id(p);
  if (epi < 0)
    return set_error("aqtx_gemm_i8: unsupported out/dequant/scale dtype combination (%d, %d, %d)",
                     p->out_dtype, p->dequant_dtype, p->row_scale_dtype);
  const bool ktail = (p->k % (2 * BK)) != 0;

  // few output tiles: the 128 x 128 kernel, with K in slices where that still leaves CUs idle
  AQTX_REQUIRE(p->k_split >= 0 && p->k_split <= 64, "aqtx_gemm_i8: k_split must be in 0..64, got %d", p->k_split);
  if (int slices = gemm_mid_k_slices(p); slices > 0) {
    // slices the library chose itself are dropped where the caller lent no (or too small a) workspace
    if (p->k_split == 0 && slices > 1 &&
        (p->k_split_workspace == nullptr || p->k_split_workspace_bytes < (int64_t)slices * p->batch * p->m * p->n * 4))
      slices = 1;
    return launch_gemm_i8_mid(p, a, b, row_scale, col_scale, c, acc_out, slices, st);
  }
  AQTX_REQUIRE(p->k_split <= 1, "aqtx_gemm_i8: k_split > 1 with ragged batches, plan->tuning or unaligned operands");
  // Two waves per SIMD by default: measured faster on every shape tried (the epilogue of one
  // wave overlaps the other's work).  plan->tuning = 4 | 8 overrides it (tests, tuning).
  if (b_frag) {
    AQTX_REQUIRE((p->tuning == 0 || p->tuning == 8) && !g.col_first,
                 "aqtx_gemm_i8: a fragment-ordered b takes scale_order AQTX_SCALE_ROW_THEN_COL and tuning 0, 8 or 128");
    return launch_gemm_i8_frag(p, a, b, row_scale, col_scale, c, acc_out, st);
  }
  const int waves = p->tuning == 4 ? 4 : 8;
  AQTX_REQUIRE(!b_packed || !g.col_first, "aqtx_gemm_i8: a packed int4 b takes scale_order = AQTX_SCALE_ROW_THEN_COL");
  // One workgroup per CU that walks the tiles (gemm_kernel's PERSIST) where there are at least two rounds of them:
  // no workgroup launch between two tiles, and the next tile's first loads pass under the epilogue's stores.
  const int cus = compute_units();
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  const bool persist = waves == 8 && !b_packed && !ktail && p->batch == 1 && p->group_offsets == nullptr && cus > 0 &&
                       (p->tuning == 16 || (p->tuning == 0 && tiles >= 2 * cus));
  const dim3 pgrid((unsigned)(tiles < cus ? tiles : cus), 1);
  // packed int4 B: the 8-wave kernel, row scale first (a frozen weight is the column operand)
#define AQTX_LAUNCH(E, C, T)                                             \
  do {                                                                  \
    if constexpr (!C) {                                                 \
      if (b_packed) { gemm_kernel<MmaI8, 8, E, false, T, true><<<grid, 512, 0, st>>>(g); break; } \
    }                                                                   \
    if constexpr (!T) {                                                 \
      if (persist) { gemm_kernel<MmaI8, 8, E, C, false, false, false, true><<<pgrid, 512, 0, st>>>(g); break; } \
    }                                                                   \
    if (waves == 8) gemm_kernel<MmaI8, 8, E, C, T><<<grid, 512, 0, st>>>(g); \
    else gemm_kernel<MmaI8, 4, E, C, T><<<grid, 256, 0, st>>>(g);       \
  } while (0)
#define AQTX_LAUNCH_T(E, C) \
  do { if (ktail) AQTX_LAUNCH(E, C, true); else AQTX_LAUNCH(E, C, false); } while (0)
#define AQTX_LAUNCH_C(E) \
  do { if (g.col_first) AQTX_LAUNCH_T(E, true); else AQTX_LAUNCH_T(E, false); } while (0)
  switch (epi) {
    case 0: AQTX_LAUNCH_C(0); break;
    case 1: AQTX_LAUNCH_C(1); break;
    case 2: AQTX_LAUNCH_C(2); break;
    case 4: AQTX_LAUNCH_C(4); break;
    default: AQTX_LAUNCH_T(3, false); break;
  }
#undef AQTX_LAUNCH_C
#undef AQTX_LAUNCH_T
#undef AQTX_LAUNCH
  AQTX_HIP_CHECK_LAUNCH("gemm_kernel<int8>");
  return 0;
}

extern "C" int aqtx_conv_i8(const aqtx_im2col_plan* w, const aqtx_gemm_plan* p, const void* x, const void* b,
                            const float* row_scale, const float* col_scale, void* c, void* stream) {
  clear_error();
  AQTX_REQUIRE(w != nullptr, "aqtx_conv_i8: window plan is NULL");
  if (int rc = validate_gemm_plan(p, "aqtx_conv_i8", false)) return rc;
  AQTX_REQUIRE(w->rank >= 1 && w->rank <= 3, "aqtx_conv_i8: spatial rank %d outside 1..3", w->rank);
  AQTX_REQUIRE(w->n >= 0 && w->c >= 0, "aqtx_conv_i8: negative shape");
  int64_t positions = 1, taps = 1, in_elems = 1;
  for (int d = 0; d < w->rank; ++d) {
    AQTX_REQUIRE(w->in_size[d] >= 0 && w->kernel[d] >= 1 && w->stride[d] >= 1 && w->dilation[d] >= 1 &&
                     w->pad_lo[d] >= 0 && w->out_size[d] >= 0,
                 "aqtx_conv_i8: bad extent on spatial axis %d", d);
    positions *= w->out_size[d];
    taps *= w->kernel[d];
    in_elems *= w->in_size[d];
  }
  AQTX_REQUIRE(p->batch == 1 && p->m == w->n * positions && p->k == taps * w->c && p->group_offsets == nullptr,
               "aqtx_conv_i8: the contraction plan must be batch 1, m = images * positions, k = taps * features");
  AQTX_REQUIRE(p->a_dtype != AQTX_I4P && p->b_dtype != AQTX_I4P && p->out_dtype != AQTX_I32 && p->k_split <= 1,
               "aqtx_conv_i8: int8 containers, a float output and no k slices");
  if (p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(x != nullptr && b != nullptr && c != nullptr, "aqtx_conv_i8: NULL buffer");
  AQTX_REQUIRE(w->c > 0 && w->c % 128 == 0, "aqtx_conv_i8: features (%d) must be a positive multiple of 128 "
               "(other inputs go through aqtx_im2col_i8 + aqtx_gemm_i8)", w->c);
  AQTX_REQUIRE(w->n * in_elems * w->c < (1ll << 31), "aqtx_conv_i8: input of 2 GiB or more");
  AQTX_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)b % 16) == 0 && p->ldb % 16 == 0 && p->ldb * (int64_t)128 < (1ll << 31),
               "aqtx_conv_i8: operands must be 16-byte aligned, ldb a multiple of 16");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)c % esz) == 0, "aqtx_conv_i8: output is not element aligned");
  return launch_conv_i8_mid(w, p, x, b, row_scale, col_scale, c, reinterpret_cast<hipStream_t>(stream));
}

extern "C" int aqtx_gemm_weight_only(const aqtx_gemm_plan* p, const void* a, const void* b, const float* col_scale,
                                     void* c, void* stream) {
  clear_error();
  const char* who = "aqtx_gemm_weight_only";
  AQTX_REQUIRE(p != nullptr, "%s: plan is NULL", who);
  AQTX_REQUIRE(p->batch >= 0 && p->m >= 0 && p->n >= 0 && p->k >= 0, "%s: negative shape", who);
  AQTX_REQUIRE(p->a_dtype == AQTX_BF16 && (p->b_dtype == AQTX_I8 || p->b_dtype == AQTX_I4),
               "%s: a must be bf16 and b int8 containers (got %d, %d)", who, p->a_dtype, p->b_dtype);
  AQTX_REQUIRE(p->out_dtype == AQTX_BF16 && p->dequant_dtype == AQTX_BF16, "%s: out_dtype and dequant_dtype must be bf16", who);
  AQTX_REQUIRE(is_float_dtype(p->col_scale_dtype), "%s: col_scale_dtype must be bf16 or f32", who);
  AQTX_REQUIRE(p->group_offsets == nullptr && p->k_split <= 1, "%s: no ragged batches, no slices of k", who);
  const bool b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  AQTX_REQUIRE(p->b_layout == AQTX_W_ROWS || (b_frag && p->batch <= 1), "%s: b_layout must be AQTX_W_ROWS, or AQTX_W_FRAGMENTS with batch 1", who);
  AQTX_REQUIRE(!b_frag || ((p->n + 15) / 16) * ((p->k + 63) / 64) * 1024 < (1ll << 31), "%s: fragment-ordered weight larger than 2 GiB", who);
  AQTX_REQUIRE(p->lda >= p->k && (b_frag || p->ldb >= p->k) && p->ldc >= p->n, "%s: leading dimension smaller than the row length", who);
  AQTX_REQUIRE(p->k > 0 && p->k % 16 == 0, "%s: k = %lld must be a positive multiple of 16", who, (long long)p->k);
  AQTX_REQUIRE(p->lda % 8 == 0 && p->stride_a % 8 == 0 && (b_frag || (p->ldb % 16 == 0 && p->stride_b % 16 == 0)),
               "%s: rows of a and b must start 16-byte aligned", who);
  AQTX_REQUIRE(p->batch <= 65535 && p->m <= (int64_t)65535 * 128 && (p->m + 127) / 128 * ((p->n + 127) / 128) < (1ll << 31),
               "%s: shape too large for one launch", who);
  AQTX_REQUIRE(p->lda * 256 < (1ll << 31) && (b_frag || p->ldb * 256 < (1ll << 31)), "%s: leading dimension too large for 32-bit tile offsets", who);
  if (p->batch == 0 || p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "%s: NULL buffer", who);
  AQTX_REQUIRE(((uintptr_t)a % 16) == 0 && ((uintptr_t)b % 16) == 0 && ((uintptr_t)c % 2) == 0, "%s: a and b must be 16-byte aligned", who);
  // 256 x 256 tiles where they fill the chip (the rule of aqtx_gemm_i8), walked by one workgroup per CU from two
  // rounds of them on; plan->tuning: 128 = the 128 x 128 tiles, 8 = the large ones with a workgroup per tile
  const int64_t pad256 = ((p->m + BM - 1) / BM) * ((p->n + BN - 1) / BN), pad128 = ((p->m + 127) / 128) * ((p->n + 127) / 128);
  const bool large = p->tuning == 8 || p->tuning == 16 ||
                     (p->tuning == 0 && pad256 * p->batch > 128 && 4 * pad256 * 2 < 3 * pad128);
  if (large && p->lda * (int64_t)(2 * BM) < (1ll << 31) && (b_frag || p->ldb * (int64_t)BN < (1ll << 31))) {
    const int cus = compute_units();
    const int workgroups = (p->tuning == 16 || (p->tuning == 0 && pad256 >= 2 * cus)) ? cus : 0;
    return launch_gemm_weight_only_large(p, a, b, col_scale, c, workgroups, reinterpret_cast<hipStream_t>(stream));
  }
  return launch_gemm_weight_only_mid(p, a, b, col_scale, c, reinterpret_cast<hipStream_t>(stream));
}

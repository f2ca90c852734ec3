// fp8 x fp8 -> float32 contraction on gfx950 MFMA (v_mfma_scale_f32_32x32x64_f8f6f4 with
// unit block scales) with the dequantisation fused in the epilogue; the kernel lives in
// gemm_core.h.  Each operand is e4m3fn or e5m2 independently.  plan->accumulate == AQTX_ACC_F32
// sends the plan through bf16 instead (gemm_mid.hip, MmaBf16F8).
#include "gemm_core.h"

using namespace aqtx;

namespace {

template <class MMA>
int launch_fp8(const GemmArgs& g, int epi, dim3 grid, hipStream_t st) {
  // K tails are always masked here: fewer instantiations, and the mask is one compare per load.
#define AQTX_LAUNCH(E, C) gemm_kernel<MMA, 8, E, C, true><<<grid, 512, 0, st>>>(g)
#define AQTX_LAUNCH_C(E) do { if (g.col_first) AQTX_LAUNCH(E, true); else AQTX_LAUNCH(E, false); } while (0)
  switch (epi) {
    case 0: AQTX_LAUNCH_C(0); break;
    case 1: AQTX_LAUNCH_C(1); break;
    case 4: AQTX_LAUNCH_C(4); break;
    default: AQTX_LAUNCH_C(2); break;
  }
#undef AQTX_LAUNCH_C
#undef AQTX_LAUNCH
  AQTX_HIP_CHECK_LAUNCH("gemm_kernel<fp8>");
  return 0;
}

}  // namespace

extern "C" int aqtx_gemm_fp8(const aqtx_gemm_plan* p, const void* a, const void* b,
                             const float* row_scale, const float* col_scale, void* c,
                             float* acc_out, void* stream) {
  clear_error();
  if (int rc = validate_gemm_plan(p, "aqtx_gemm_fp8", true)) return rc;
  if (p->batch == 0 || p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "aqtx_gemm_fp8: NULL buffer");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)c % esz) == 0, "aqtx_gemm_fp8: output is not element aligned");

  const GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool a5 = p->a_dtype == AQTX_E5M2, b5 = p->b_dtype == AQTX_E5M2;

  if (!gemm_vector_path_ok(p, a, b)) {
    AQTX_REQUIRE(p->group_offsets == nullptr, "aqtx_gemm_fp8: ragged batches need aligned operands");
    dim3 grid((unsigned)((p->n + 255) / 256), (unsigned)p->m, (unsigned)p->batch);
    AQTX_REQUIRE(p->m <= 65535, "aqtx_gemm_fp8: m too large for the unaligned path");
    if (!a5 && !b5) gemm_simple_kernel<DecE4M3, DecE4M3, false><<<grid, 256, 0, st>>>(g);
    else if (!a5 && b5) gemm_simple_kernel<DecE4M3, DecE5M2, false><<<grid, 256, 0, st>>>(g);
    else if (a5 && !b5) gemm_simple_kernel<DecE5M2, DecE4M3, false><<<grid, 256, 0, st>>>(g);
    else gemm_simple_kernel<DecE5M2, DecE5M2, false><<<grid, 256, 0, st>>>(g);
    AQTX_HIP_CHECK_LAUNCH("gemm_simple_kernel");
    return 0;
  }
  if (p->accumulate == AQTX_ACC_F32) return launch_gemm_fp8_f32sum_mid(p, a, b, row_scale, col_scale, c, acc_out, st);
  // few output tiles (or tiles that would lie mostly outside C): the 128 x 128 kernel
  if (p->k_split <= 1 && gemm_mid_k_slices(p) > 0) return launch_gemm_fp8_mid(p, a, b, row_scale, col_scale, c, acc_out, st);
  AQTX_REQUIRE(p->lda * (int64_t)BM < (1ll << 31) && p->ldb * (int64_t)BN < (1ll << 31),
               "aqtx_gemm_fp8: leading dimension too large for 32-bit tile offsets");
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  const int epi = gemm_epilogue_id(p);
  if (epi < 0 || epi == 3)
    return set_error("aqtx_gemm_fp8: unsupported out/dequant/scale dtype combination (%d, %d, %d)",
                     p->out_dtype, p->dequant_dtype, p->row_scale_dtype);
  if (!a5 && !b5) return launch_fp8<MmaF8<0, 0>>(g, epi, grid, st);
  if (!a5 && b5) return launch_fp8<MmaF8<0, 1>>(g, epi, grid, st);
  if (a5 && !b5) return launch_fp8<MmaF8<1, 0>>(g, epi, grid, st);
  return launch_fp8<MmaF8<1, 1>>(g, epi, grid, st);
}

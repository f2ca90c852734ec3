// aqtx_gemm_weight_only on 256 x 256 tiles: gemm_kernel with bf16 rows of A, the int8 rows of B loaded as the
// packed int4 variant loads them (16 rows x 64 bytes per wave load) and widened to bf16, exactly, on their way to
// LDS, and v_mfma_f32_32x32x16_bf16; float32 sums.  For shapes with many output tiles; the few-tile shapes stay
// with the 128 x 128 kernel (gemm_mid.hip).  In a file of its own so that it compiles next to the others.
#include "gemm_core.h"

namespace aqtx {

int launch_gemm_weight_only_large(const aqtx_gemm_plan* p, const void* a, const void* b, const float* col_scale, void* c,
                                  int workgroups, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, nullptr, col_scale, c, nullptr);
  g.k *= 2; g.lda *= 2; g.stride_a *= 2;  // A in bytes; a 128-byte stage is 64 k
  g.col_first = 0;
  g.b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  g.b_steps = (int)((p->k + 63) / 64);
  const bool ktail = (g.k % (2 * BK)) != 0;
  const bool f32_scale = p->col_scale_dtype != AQTX_BF16;  // epilogue 4: first product bf16 (no row scale), second f32
  const int64_t tiles = (int64_t)g.tiles_m * g.tiles_n;
  const bool persist = workgroups > 0 && !ktail && p->batch == 1;
  const dim3 grid(persist ? (unsigned)(tiles < workgroups ? tiles : workgroups) : (unsigned)tiles, (unsigned)p->batch);
#define AQTX_WO(E, FRAG)                                                                                       \
  do {                                                                                                         \
    if (persist) gemm_kernel<MmaBf16W8, 8, E, false, false, true, FRAG, true><<<grid, 512, 0, st>>>(g);        \
    else if (ktail) gemm_kernel<MmaBf16W8, 8, E, false, true, true, FRAG><<<grid, 512, 0, st>>>(g);            \
    else gemm_kernel<MmaBf16W8, 8, E, false, false, true, FRAG><<<grid, 512, 0, st>>>(g);                      \
  } while (0)
  if (g.b_frag) { if (f32_scale) AQTX_WO(4, true); else AQTX_WO(0, true); }
  else { if (f32_scale) AQTX_WO(4, false); else AQTX_WO(0, false); }
#undef AQTX_WO
  AQTX_HIP_CHECK_LAUNCH("gemm_kernel<weight only>");
  return 0;
}

}  // namespace aqtx

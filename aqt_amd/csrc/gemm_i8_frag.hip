// aqtx_gemm_i8 on 256 x 256 tiles with b in the fragment order of aqtx_tile_weight: the instantiations of
// gemm_kernel<..., BFRAG> (8 waves, row scale first), in a file of their own so that they compile next to
// the others.  The kernel differs from the one that reads rows in the addresses of its B loads only.
#include "gemm_core.h"

namespace aqtx {

int launch_gemm_i8_frag(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                        const float* col_scale, void* c, int32_t* acc_out, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  const bool packed = p->b_dtype == AQTX_I4P;
  g.a_even_odd8 = p->a_k_order == AQTX_K_EVEN_ODD8;
  g.b_frag = 1;
  g.b_steps = (int)(((packed ? p->k / 2 : p->k) + 63) / 64);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  const int epi = gemm_epilogue_id(p);
  const bool ktail = (p->k % (2 * BK)) != 0;
#define AQTX_FRAG(E)                                                                                        \
  do {                                                                                                      \
    if (packed) {                                                                                           \
      if (ktail) gemm_kernel<MmaI8, 8, E, false, true, true, true><<<grid, 512, 0, st>>>(g);               \
      else gemm_kernel<MmaI8, 8, E, false, false, true, true><<<grid, 512, 0, st>>>(g);                    \
    } else {                                                                                                \
      if (ktail) gemm_kernel<MmaI8, 8, E, false, true, false, true><<<grid, 512, 0, st>>>(g);              \
      else gemm_kernel<MmaI8, 8, E, false, false, false, true><<<grid, 512, 0, st>>>(g);                   \
    }                                                                                                       \
  } while (0)
  switch (epi) {
    case 0: AQTX_FRAG(0); break;
    case 1: AQTX_FRAG(1); break;
    case 2: AQTX_FRAG(2); break;
    case 4: AQTX_FRAG(4); break;
    default: AQTX_FRAG(3); break;
  }
#undef AQTX_FRAG
  AQTX_HIP_CHECK_LAUNCH("gemm_kernel<int8, fragment-ordered b>");
  return 0;
}

}  // namespace aqtx

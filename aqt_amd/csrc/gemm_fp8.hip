// fp8 x fp8 -> float32 contraction (placeholder until the MFMA kernel lands).
#include "common.h"
using namespace aqtx;
extern "C" int aqtx_gemm_fp8(const aqtx_gemm_plan*, const void*, const void*, const float*,
                             const float*, void*, float*, void*) {
  return set_error("aqtx_gemm_fp8: not implemented in this build");
}

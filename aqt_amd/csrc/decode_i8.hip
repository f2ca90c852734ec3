// Serving-shape contraction (placeholder until the kernel lands).
#include "common.h"
using namespace aqtx;
extern "C" size_t aqtx_decode_workspace_bytes(const aqtx_decode_plan*) { return 0; }
extern "C" int aqtx_decode_i8(const aqtx_decode_plan*, const void*, const void*, const float*, void*,
                              float*, void*, void*, size_t, void*) {
  return set_error("aqtx_decode_i8: not implemented in this build");
}

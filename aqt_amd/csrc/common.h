// Shared host/device helpers of the aqtx kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>
#include "../../include/aqtx.h"

namespace aqtx {

// ---- error reporting -------------------------------------------------------
int set_error(const char* fmt, ...);
void clear_error();

#define AQTX_REQUIRE(cond, ...)                 \
  do {                                          \
    if (!(cond)) return ::aqtx::set_error(__VA_ARGS__); \
  } while (0)

#define AQTX_HIP_CHECK_LAUNCH(name)                                            \
  do {                                                                         \
    hipError_t e__ = hipGetLastError();                                        \
    if (e__ != hipSuccess)                                                     \
      return ::aqtx::set_error("%s: launch failed: %s", name, hipGetErrorString(e__)); \
  } while (0)

inline bool is_float_dtype(int d) { return d == AQTX_F32 || d == AQTX_BF16; }
inline size_t dtype_size(int d) {
  switch (d) {
    case AQTX_F32: case AQTX_I32: return 4;
    case AQTX_BF16: return 2;
    default: return 1;
  }
}

// ---- device numerics -------------------------------------------------------
#if defined(__HIPCC__)

// Cache policy argument of a raw buffer load for bytes a launch reads once, in whole cache lines per wave
// load (a fragment-ordered weight streamed past many activations): the non-temporal hint keeps them from
// displacing what is re-read from the L2.  Measured on the serving kernels: 5-12 % off a call.  Not for
// loads that take half a line at a time (weight rows): their other half would be fetched twice.
constexpr int kStreamOnce = 2;

// float -> nearest bf16 (ties to even), returned as float.
__device__ __forceinline__ float round_bf16(float x) {
  return (float)(__bf16)x;
}
__device__ __forceinline__ uint16_t bf16_bits(float x) {
  __bf16 h = (__bf16)x;
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
// Running abs-max that keeps a NaN, as jnp.max(jnp.abs(x)) does (aqt/jax/v2/calibration.py:126): a
// diverged step must show up as a NaN scale and NaN outputs, and v_max_f32 would drop it.  For
// non-negative floats and NaNs (sign cleared) the unsigned order of the bit patterns is the order
// wanted: every NaN pattern lies above infinity.
__device__ __forceinline__ float nanmax(float a, float b) {  // a, b: non-negative or NaN
  const uint32_t x = __float_as_uint(a), y = __float_as_uint(b);
  return __uint_as_float(x > y ? x : y);
}
__device__ __forceinline__ float absmax_step(float m, float v) {  // max(m, |v|)
  return nanmax(m, __uint_as_float(__float_as_uint(v) & 0x7FFFFFFFu));
}

// Round to the dtype tag (AQTX_BF16 rounds, AQTX_F32 is the identity).
template <bool kBf16>
__device__ __forceinline__ float round_to(float x) {
  if constexpr (kBf16) return round_bf16(x);
  return x;
}

#endif  // __HIPCC__

}  // namespace aqtx

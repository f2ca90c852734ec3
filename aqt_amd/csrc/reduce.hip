// Sum of per-tile partial results over a leading axis, the last step of a tiled dot_general:
// out[i] = cast( sum_t float(x[t][i]) ), accumulated in float32 in tile order and rounded once,
// which is what jnp.sum does for 16-bit floats.  One pass over x; HBM-bound.
#include "common.h"

namespace aqtx {
namespace {

template <bool BF16>
__global__ __launch_bounds__(256) void sum_tiles_kernel(const void* x, void* out, int64_t tiles, int64_t count) {
  constexpr int VEC = BF16 ? 8 : 4;  // 16 bytes per lane and tile
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (i0 >= count) return;
  float acc[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) acc[e] = 0.0f;
  if (i0 + VEC <= count && (count % VEC) == 0) {
    for (int64_t t = 0; t < tiles; ++t) {
      if constexpr (BF16) {
        const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(x) + t * count + i0);
        const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          acc[2 * e] += __uint_as_float(w[e] << 16);
          acc[2 * e + 1] += __uint_as_float(w[e] & 0xFFFF0000u);
        }
      } else {
        const float4 v = *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(x) + t * count + i0);
        acc[0] += v.x; acc[1] += v.y; acc[2] += v.z; acc[3] += v.w;
      }
    }
    if constexpr (BF16) {
      uint4 o;
      o.x = bf16_bits(acc[0]) | ((uint32_t)bf16_bits(acc[1]) << 16);
      o.y = bf16_bits(acc[2]) | ((uint32_t)bf16_bits(acc[3]) << 16);
      o.z = bf16_bits(acc[4]) | ((uint32_t)bf16_bits(acc[5]) << 16);
      o.w = bf16_bits(acc[6]) | ((uint32_t)bf16_bits(acc[7]) << 16);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(out) + i0) = o;
    } else {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(out) + i0) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    }
    return;
  }
  // ragged tail or a row length that breaks the 16-byte alignment of later tiles
  for (int e = 0; e < VEC && i0 + e < count; ++e) {
    float a = 0.0f;
    for (int64_t t = 0; t < tiles; ++t) {
      if constexpr (BF16) a += bf16_bits_to_float(reinterpret_cast<const uint16_t*>(x)[t * count + i0 + e]);
      else a += reinterpret_cast<const float*>(x)[t * count + i0 + e];
    }
    if constexpr (BF16) reinterpret_cast<uint16_t*>(out)[i0 + e] = bf16_bits(a);
    else reinterpret_cast<float*>(out)[i0 + e] = a;
  }
}

// Reads `bytes` once, 16 bytes per lane and load (with the non-temporal hint the serving kernels give
// their weight loads), PER loads in flight per lane, and writes one word per workgroup: the least any
// kernel that streams a buffer of this size can take.
template <int PER>
__global__ __launch_bounds__(256) void read_probe_kernel(const uint4* p, int64_t vecs, uint32_t* out) {
  uint32_t acc = 0u;
  const int64_t base = (int64_t)blockIdx.x * 256 * PER + threadIdx.x;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int64_t i = base + (int64_t)j * 256;
    if (i < vecs) {
      typedef unsigned int v4u __attribute__((ext_vector_type(4)));
      const v4u v = __builtin_nontemporal_load(reinterpret_cast<const v4u*>(p + i));
      acc ^= v[0] ^ v[1] ^ v[2] ^ v[3];
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) acc ^= __shfl_xor(acc, off, 64);
  if ((threadIdx.x & 63) == 0) atomicXor(out + blockIdx.x, acc);
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_read_probe(const void* src, int64_t bytes, void* out_words, int64_t out_count, void* stream) {
  clear_error();
  AQTX_REQUIRE(bytes >= 0 && bytes % 16 == 0, "aqtx_read_probe: bytes must be a non-negative multiple of 16");
  if (bytes == 0) return 0;
  AQTX_REQUIRE(src != nullptr && out_words != nullptr, "aqtx_read_probe: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)src % 16) == 0, "aqtx_read_probe: src must be 16-byte aligned");
  constexpr int kPer = 16;  // 64 KiB per workgroup
  const int64_t vecs = bytes / 16;
  const int64_t blocks = (vecs + 256 * kPer - 1) / (256 * kPer);
  AQTX_REQUIRE(blocks <= out_count && blocks < (1ll << 31), "aqtx_read_probe: out needs %lld words", (long long)blocks);
  read_probe_kernel<kPer><<<(unsigned)blocks, 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint4*>(src), vecs, reinterpret_cast<uint32_t*>(out_words));
  AQTX_HIP_CHECK_LAUNCH("read_probe_kernel");
  return 0;
}

extern "C" int aqtx_sum_tiles(const void* x, void* out, int64_t tiles, int64_t count, int32_t dtype,
                              void* stream) {
  clear_error();
  AQTX_REQUIRE(tiles >= 0 && count >= 0, "aqtx_sum_tiles: negative shape");
  AQTX_REQUIRE(is_float_dtype(dtype), "aqtx_sum_tiles: dtype must be bf16 or f32, got %d", dtype);
  if (count == 0) return 0;
  AQTX_REQUIRE(x != nullptr && out != nullptr, "aqtx_sum_tiles: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0,
               "aqtx_sum_tiles: x and out must be 16-byte aligned");
  const int vec = dtype == AQTX_BF16 ? 8 : 4;
  const int64_t blocks = (count + 256 * vec - 1) / (256 * vec);
  AQTX_REQUIRE(blocks < (1ll << 31), "aqtx_sum_tiles: count too large for one launch");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (dtype == AQTX_BF16) sum_tiles_kernel<true><<<(unsigned)blocks, 256, 0, st>>>(x, out, tiles, count);
  else sum_tiles_kernel<false><<<(unsigned)blocks, 256, 0, st>>>(x, out, tiles, count);
  AQTX_HIP_CHECK_LAUNCH("sum_tiles_kernel");
  return 0;
}

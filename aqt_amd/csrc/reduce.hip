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

// Reads `bytes` once and does nothing else.  A workgroup of 256 lanes takes chunks of 256 * U * 16 bytes, chunk
// c = blockIdx.x + i * gridDim.x (a grid of as many workgroups as chunks reads one chunk each), U loads of 16
// bytes per lane in flight, each wave load one contiguous KiB; POLICY is the cache policy of the buffer loads
// (bit 1 = the non-temporal hint the serving kernels give their weight loads).  One checksum word per
// workgroup leaves, and, where asked for, the workgroup's first and last reading of the device's constant-rate
// clock, from which the host takes the span of the launch without the time to launch it.
template <int U, int POLICY>
__global__ __launch_bounds__(256) void read_probe_kernel(const uint8_t* src, uint32_t bytes, int nchunks, uint32_t* out,
                                                         unsigned long long* stamps) {
  typedef int v4i __attribute__((ext_vector_type(4)));
  const int tid = threadIdx.x;
  unsigned long long t0 = 0;
  if (stamps != nullptr && tid == 0) t0 = wall_clock64();
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc((void*)src, 0, (int)bytes, 0x00020000u);
  v4i acc = {0, 0, 0, 0};
  for (int c = blockIdx.x; c < nchunks; c += gridDim.x) {
    const uint32_t cb = (uint32_t)c * (256u * U * 16u);
    v4i v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, tid * 16 + u * 4096, cb, POLICY);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  uint32_t x = (uint32_t)(acc[0] ^ acc[1] ^ acc[2] ^ acc[3]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) x ^= __shfl_xor(x, off, 64);
  if ((tid & 63) == 0) atomicXor(out + blockIdx.x, x);
  if (stamps != nullptr && tid == 0) {
    stamps[2 * blockIdx.x] = t0;
    stamps[2 * blockIdx.x + 1] = wall_clock64();
  }
}

template <int POLICY>
void launch_read_probe(int loads, dim3 grid, hipStream_t st, const uint8_t* src, uint32_t bytes, int nchunks, uint32_t* out,
                       unsigned long long* stamps) {
  switch (loads) {
    case 2: read_probe_kernel<2, POLICY><<<grid, 256, 0, st>>>(src, bytes, nchunks, out, stamps); break;
    case 4: read_probe_kernel<4, POLICY><<<grid, 256, 0, st>>>(src, bytes, nchunks, out, stamps); break;
    case 8: read_probe_kernel<8, POLICY><<<grid, 256, 0, st>>>(src, bytes, nchunks, out, stamps); break;
    default: read_probe_kernel<16, POLICY><<<grid, 256, 0, st>>>(src, bytes, nchunks, out, stamps); break;
  }
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_read_probe(const void* src, int64_t bytes, int32_t workgroups, int32_t loads_in_flight,
                               int32_t cache_policy, void* out_words, uint64_t* stamps, int32_t* wall_clock_khz,
                               void* stream) {
  clear_error();
  AQTX_REQUIRE(bytes >= 0 && bytes % 16 == 0 && bytes < (1ll << 31), "aqtx_read_probe: bytes must be a multiple of 16 below 2 GiB");
  AQTX_REQUIRE(loads_in_flight == 2 || loads_in_flight == 4 || loads_in_flight == 8 || loads_in_flight == 16,
               "aqtx_read_probe: loads_in_flight must be 2, 4, 8 or 16");
  AQTX_REQUIRE(cache_policy >= 0 && cache_policy <= 3, "aqtx_read_probe: cache_policy must be 0..3");
  AQTX_REQUIRE(workgroups >= 0 && workgroups <= 65536, "aqtx_read_probe: at most 65536 workgroups");
  if (wall_clock_khz != nullptr) {
    int dev = 0, khz = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess)
      return set_error("aqtx_read_probe: the device does not report its wall clock rate");
    *wall_clock_khz = khz;
  }
  if (bytes == 0) return 0;
  AQTX_REQUIRE(src != nullptr && out_words != nullptr, "aqtx_read_probe: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)src % 16) == 0, "aqtx_read_probe: src must be 16-byte aligned");
  const int64_t chunk = 256ll * loads_in_flight * 16;
  const int64_t nchunks = (bytes + chunk - 1) / chunk;
  int64_t grid = workgroups == 0 ? nchunks : workgroups;
  if (grid > nchunks) grid = nchunks;
  AQTX_REQUIRE(grid <= 65536, "aqtx_read_probe: %lld chunks need a workgroup count (at most 65536 workgroups write words)",
               (long long)nchunks);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const uint8_t* p = reinterpret_cast<const uint8_t*>(src);
  uint32_t* out = reinterpret_cast<uint32_t*>(out_words);
  unsigned long long* ts = reinterpret_cast<unsigned long long*>(stamps);
  switch (cache_policy) {
    case 0: launch_read_probe<0>(loads_in_flight, dim3((unsigned)grid), st, p, (uint32_t)bytes, (int)nchunks, out, ts); break;
    case 1: launch_read_probe<1>(loads_in_flight, dim3((unsigned)grid), st, p, (uint32_t)bytes, (int)nchunks, out, ts); break;
    case 2: launch_read_probe<2>(loads_in_flight, dim3((unsigned)grid), st, p, (uint32_t)bytes, (int)nchunks, out, ts); break;
    default: launch_read_probe<3>(loads_in_flight, dim3((unsigned)grid), st, p, (uint32_t)bytes, (int)nchunks, out, ts); break;
  }
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

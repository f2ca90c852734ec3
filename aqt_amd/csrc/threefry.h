// Threefry-2x32-20 and the jax.random counter layouts, shared by host and device code.
//
// jax.random (third-party to the reference, which calls it at
// aqt/jax/v2/config.py:61-63, stochastic_rounding.py:46,65 and
// numerics/fp8_numerics.py:54) draws every bit from this block function
// (Salmon et al., SC'11).  Two counter layouts exist upstream:
//   original      : the n counters 0..n-1 are split in halves that feed the two
//                   lanes; word i < half is lane 0 of block (i, i+half), word
//                   i >= half is lane 1 of block (i-half, i); an odd n pads one 0.
//   partitionable : element i uses block (hi32(i), lo32(i)); a 32-bit draw is
//                   lane0 ^ lane1, narrower draws truncate it.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define AQTX_HD __host__ __device__ __forceinline__
#else
#define AQTX_HD inline
#endif

namespace aqtx {

struct U2 { uint32_t x, y; };

AQTX_HD uint32_t rotl32(uint32_t v, int r) { return (v << r) | (v >> (32 - r)); }

AQTX_HD U2 threefry2x32(uint32_t k0, uint32_t k1, uint32_t c0, uint32_t c1) {
  const uint32_t k2 = k0 ^ k1 ^ 0x1BD11BDAu;
  uint32_t x0 = c0 + k0, x1 = c1 + k1;
#define AQTX_TF_ROUND(r) x0 += x1; x1 = rotl32(x1, r); x1 ^= x0;
  AQTX_TF_ROUND(13) AQTX_TF_ROUND(15) AQTX_TF_ROUND(26) AQTX_TF_ROUND(6)
  x0 += k1; x1 += k2 + 1u;
  AQTX_TF_ROUND(17) AQTX_TF_ROUND(29) AQTX_TF_ROUND(16) AQTX_TF_ROUND(24)
  x0 += k2; x1 += k0 + 2u;
  AQTX_TF_ROUND(13) AQTX_TF_ROUND(15) AQTX_TF_ROUND(26) AQTX_TF_ROUND(6)
  x0 += k0; x1 += k1 + 3u;
  AQTX_TF_ROUND(17) AQTX_TF_ROUND(29) AQTX_TF_ROUND(16) AQTX_TF_ROUND(24)
  x0 += k1; x1 += k2 + 4u;
  AQTX_TF_ROUND(13) AQTX_TF_ROUND(15) AQTX_TF_ROUND(26) AQTX_TF_ROUND(6)
  x0 += k2; x1 += k0 + 5u;
#undef AQTX_TF_ROUND
  return U2{x0, x1};
}

// Generator for a flat noise tensor of `total` elements drawn `width` bits each.
struct BitGen {
  uint32_t k0, k1;
  uint32_t nwords;  // original layout: number of 32-bit words generated
  uint32_t half;    // original layout: ceil(nwords / 2)
  int32_t partitionable;
  int32_t width;    // 16 or 32

  // word `w` of the original layout
  AQTX_HD uint32_t word_original(uint32_t w) const {
    if (w < half) {
      uint32_t c1 = w + half;
      c1 = (c1 < nwords) ? c1 : 0u;
      return threefry2x32(k0, k1, w, c1).x;
    }
    return threefry2x32(k0, k1, w - half, w).y;
  }

  // the draw of element `i` (row-major index in the noise tensor), zero-extended
  AQTX_HD uint32_t draw(uint64_t i) const {
    if (partitionable) {
      U2 b = threefry2x32(k0, k1, (uint32_t)(i >> 32), (uint32_t)i);
      uint32_t v = b.x ^ b.y;
      return width == 16 ? (v & 0xFFFFu) : v;
    }
    if (width == 16) {
      uint32_t w = word_original((uint32_t)(i >> 1));
      return (i & 1) ? (w >> 16) : (w & 0xFFFFu);
    }
    return word_original((uint32_t)i);
  }
};

inline BitGen make_bitgen(const uint32_t key[2], int64_t total, int width, int partitionable) {
  BitGen g;
  g.k0 = key[0];
  g.k1 = key[1];
  uint64_t nwords = ((uint64_t)total * (uint64_t)width + 31u) / 32u;
  g.nwords = (uint32_t)nwords;
  g.half = (uint32_t)((nwords + 1u) / 2u);
  g.partitionable = partitionable;
  g.width = width;
  return g;
}

}  // namespace aqtx

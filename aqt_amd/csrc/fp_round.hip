// Rounding to an emulated small float (e2m1, e3m0, the OCP fp4/fp5/fp6 formats ...) held in a
// bf16 or f32 container: fp_numerics.radix2_round (aqt/jax/v2/numerics/fp_numerics.py:300-459),
// and to the powers of 4 of the RADIX4 format (radix4_round, :661-706; round_radix4 below).
// Elementwise on the bit patterns: add half a truncated ulp (or masked random bits) to the
// pattern, clear the truncated mantissa bits, clamp the magnitude pattern between the smallest
// and largest normal value; magnitudes below the smallest normal are rounded linearly
// (formats with subnormals) or to +-1 (formats without).  One read and one write per element;
// HBM-bound when deterministic, threefry-bound with random bits (one block per four elements
// in the paired kernel, per two otherwise).
#include "common.h"
#include <type_traits>
#include "threefry.h"

namespace aqtx {
namespace {

struct FpArgs {
  const void* x;
  void* out;
  int64_t count;
  int64_t noise_mod;
  uint32_t trunc, trunc_mask, min_repr, max_repr;
  int32_t nmant, sub, nexp0, mode, radix4;
  float scale, inv_scale, max_sub, min_float;
  BitGen gen;
};

// floor(log4(z)) of a non-negative float32 from its exponent field: floor(floor(log2 z) / 2).  Zero and
// float32 subnormals come out far below the smallest radix-4 value, infinity and NaN far above.
__device__ __forceinline__ int floor_log4(float z) {
  return ((int)((__float_as_uint(z) >> 23) & 0xFFu) - 127) >> 1;
}

// radix4_round (aqt/jax/v2/numerics/fp_numerics.py:661-706) on a bf16 pattern; rnd = 16 random bits.
__device__ __forceinline__ uint32_t round_radix4(uint32_t ob, uint32_t rnd, const FpArgs& a) {
  const float x = __uint_as_float(ob << 16);
  if (x != x) return 0x7FC0u;
  const float ax = fabsf(x);
  float z;
  if (a.mode == AQTX_FP_NEAREST) {
    z = fabsf(1.6f * x);
  } else {
    // the bucket [4^l, 4^(l+1)) that holds |x|, its width times a uniform number in [0, 1) added to |x|
    float width = 0.0f;
    if (ax != 0.0f) {
      if (isinf(ax)) return 0x7FC0u;  // 4^inf - 4^inf in the reference
      const float lower = ldexpf(1.0f, 2 * floor_log4(ax));
      width = 4.0f * lower - lower;
    }
    const float u = __uint_as_float((rnd << 7) | 0x3F800000u) - 1.0f;
    z = ax + u * width;
  }
  const int ebit = floor_log4(z);
  if (z == 0.0f || ebit < -3) return 0u;
  const uint32_t sign = ob & 0x8000u;
  if (ebit >= 3) return sign | 0x4280u;                       // +-64
  return sign | (uint32_t)((127 + 2 * ebit) << 7);            // +-4^ebit
}

template <bool BF16>
__device__ __forceinline__ uint32_t round_pattern(uint32_t ob, uint32_t rnd, const FpArgs& a) {
  if constexpr (BF16) {
    if (a.radix4) return round_radix4(ob, rnd, a);
  }
  constexpr int CM = BF16 ? 7 : 23;
  constexpr uint32_t WRAP = BF16 ? 0xFFFFu : 0xFFFFFFFFu;
  constexpr uint32_t SIGN = BF16 ? 0x8000u : 0x80000000u;
  constexpr uint32_t MANT = (1u << CM) - 1u;
  uint32_t noise;
  if (a.mode != AQTX_FP_NEAREST) {
    noise = rnd;
    if (a.trunc > 16) noise = ((noise << 1) | 1u) << (a.trunc - 17);
    noise &= a.trunc_mask;
  } else {
    noise = 1u << (a.trunc - 1);
  }
  // unsigned addition in the container width: the carry may run into the exponent, which is
  // the next value up
  const uint32_t xb = ((ob + noise) & WRAP) & ~a.trunc_mask;
  const uint32_t mag = xb & ~SIGN;
  uint32_t out = (xb & SIGN) | min(max(mag, a.min_repr), a.max_repr);
  const float x = BF16 ? __uint_as_float(ob << 16) : __uint_as_float(ob);
  if (a.sub) {
    const uint32_t omag = min(max(ob & ~SIGN & WRAP, a.min_repr), a.max_repr);
    if ((omag & ~MANT) == a.min_repr) {
      float t = round_to<BF16>(x * a.scale);
      if (a.mode != AQTX_FP_NEAREST) {
        const float nz = (__uint_as_float((rnd << 7) | 0x3F800000u) - 1.5f) + 0x1p-17f;
        t = t + nz;
      }
      const float s = rintf(t) * a.inv_scale;
      out = BF16 ? (uint32_t)bf16_bits(s) : __float_as_uint(s);
    }
  } else if (a.mode != AQTX_FP_NEAREST) {
    const float rf = __uint_as_float((rnd << 7) | 0x40000000u) - (3.0f - 0x1p-16f);
    if (fabsf(x) < a.min_float) {
      const float r = x > rf ? 1.0f : -1.0f;
      out = BF16 ? (uint32_t)bf16_bits(r) : __float_as_uint(r);
    }
  }
  if (a.nexp0 && a.sub) {
    float v = BF16 ? __uint_as_float(out << 16) : __uint_as_float(out);
    if (v > a.max_sub) v = a.max_sub;
    if (v < -a.max_sub) v = -a.max_sub;
    out = BF16 ? (uint32_t)bf16_bits(v) : __float_as_uint(v);
  }
  return out;
}

// The 16 random bits of elements i and i + 1 (i even).
__device__ __forceinline__ void draw_pair(const FpArgs& a, int64_t i, uint32_t& r0, uint32_t& r1) {
  if (a.mode == AQTX_FP_NOISE_INDEX) {
    r0 = (uint32_t)(i % a.noise_mod) & 0xFFFFu;
    r1 = (uint32_t)((i + 1) % a.noise_mod) & 0xFFFFu;
  } else if (a.gen.partitionable) {
    r0 = a.gen.draw((uint64_t)i);
    r1 = a.gen.draw((uint64_t)i + 1);
  } else {
    const uint32_t w = a.gen.word_original((uint32_t)(i >> 1));
    r0 = w & 0xFFFFu;
    r1 = w >> 16;
  }
}

// VEC elements per lane: 16 bytes when the buffers allow it, else one pair.
template <bool BF16, int VEC>
__global__ __launch_bounds__(256) void fp_round_kernel(const FpArgs a) {
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (i0 >= a.count) return;
  uint32_t bits[VEC];
  const bool full = i0 + VEC <= a.count;
  if constexpr (VEC == 8) {
    if (full) {
      const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.x) + i0);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        bits[2 * e] = w[e] & 0xFFFFu;
        bits[2 * e + 1] = w[e] >> 16;
      }
    }
  } else if constexpr (VEC == 4) {
    if (full) {
      const uint4 v = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint32_t*>(a.x) + i0);
      bits[0] = v.x; bits[1] = v.y; bits[2] = v.z; bits[3] = v.w;
    }
  }
  if (VEC == 2 || !full) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      bits[e] = 0;
      if (i0 + e < a.count) {
        bits[e] = BF16 ? (uint32_t)reinterpret_cast<const uint16_t*>(a.x)[i0 + e]
                       : reinterpret_cast<const uint32_t*>(a.x)[i0 + e];
      }
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; e += 2) {
    uint32_t r0 = 0, r1 = 0;
    if (a.mode != AQTX_FP_NEAREST) draw_pair(a, i0 + e, r0, r1);
    bits[e] = round_pattern<BF16>(bits[e], r0, a);
    bits[e + 1] = round_pattern<BF16>(bits[e + 1], r1, a);
  }
  if constexpr (VEC == 8) {
    if (full) {
      uint4 o;
      o.x = bits[0] | (bits[1] << 16); o.y = bits[2] | (bits[3] << 16);
      o.z = bits[4] | (bits[5] << 16); o.w = bits[6] | (bits[7] << 16);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(a.out) + i0) = o;
      return;
    }
  } else if constexpr (VEC == 4) {
    if (full) {
      *reinterpret_cast<uint4*>(reinterpret_cast<uint32_t*>(a.out) + i0) = make_uint4(bits[0], bits[1], bits[2], bits[3]);
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) {
    if (i0 + e < a.count) {
      if constexpr (BF16) reinterpret_cast<uint16_t*>(a.out)[i0 + e] = (uint16_t)bits[e];
      else reinterpret_cast<uint32_t*>(a.out)[i0 + e] = bits[e];
    }
  }
}

// jax.random.bits in its original layout: one threefry block yields word w (first half of the words)
// and word w + half (second half), i.e. the 16-bit draws of elements 2w, 2w + 1 and of the two
// elements `2 * half` further on.  A lane takes VEC elements from each region so that no output
// of a block is thrown away.  Needs 2 * half to be a multiple of VEC (16-byte alignment of the
// second region).
template <bool BF16, int VEC>
__global__ __launch_bounds__(256) void fp_round_paired_kernel(const FpArgs a) {
  using T = typename std::conditional<BF16, uint16_t, uint32_t>::type;
  const int64_t second = 2 * (int64_t)a.gen.half;
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * VEC;
  if (i0 >= second) return;
  const T* x = reinterpret_cast<const T*>(a.x);
  T* out = reinterpret_cast<T*>(a.out);
  uint32_t lo[VEC], hi[VEC];
  const int64_t i1 = i0 + second;
  const bool full0 = i0 + VEC <= (second < a.count ? second : a.count);
  const bool full1 = i1 + VEC <= a.count;
  auto load = [&](int64_t base, bool full, int64_t limit, uint32_t* bits) {
    if (full) {
      const uint4 v = *reinterpret_cast<const uint4*>(x + base);
      const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if constexpr (BF16) bits[e] = (w[e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
        else bits[e] = w[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) bits[e] = base + e < limit ? (uint32_t)x[base + e] : 0u;
    }
  };
  load(i0, full0, second < a.count ? second : a.count, lo);
  load(i1, full1, a.count, hi);
#pragma unroll
  for (int e = 0; e < VEC; e += 2) {
    const uint32_t w = (uint32_t)((i0 + e) >> 1);
    uint32_t c1 = w + a.gen.half;
    c1 = c1 < a.gen.nwords ? c1 : 0u;
    const U2 blk = threefry2x32(a.gen.k0, a.gen.k1, w, c1);
    lo[e] = round_pattern<BF16>(lo[e], blk.x & 0xFFFFu, a);
    lo[e + 1] = round_pattern<BF16>(lo[e + 1], blk.x >> 16, a);
    hi[e] = round_pattern<BF16>(hi[e], blk.y & 0xFFFFu, a);
    hi[e + 1] = round_pattern<BF16>(hi[e + 1], blk.y >> 16, a);
  }
  auto store = [&](int64_t base, bool full, int64_t limit, const uint32_t* bits) {
    if (full) {
      uint4 o;
      if constexpr (BF16) {
        o = make_uint4(bits[0] | (bits[1] << 16), bits[2] | (bits[3] << 16), bits[4] | (bits[5] << 16),
                       bits[6] | (bits[7] << 16));
      } else {
        o = make_uint4(bits[0], bits[1], bits[2], bits[3]);
      }
      *reinterpret_cast<uint4*>(out + base) = o;
    } else {
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (base + e < limit) out[base + e] = (T)bits[e];
      }
    }
  };
  store(i0, full0, second < a.count ? second : a.count, lo);
  store(i1, full1, a.count, hi);
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_fp_round(const aqtx_fp_round_plan* p, const void* x, void* out,
                             const uint32_t key_host[2], void* stream) {
  clear_error();
  AQTX_REQUIRE(p != nullptr, "aqtx_fp_round: plan is NULL");
  AQTX_REQUIRE(is_float_dtype(p->dtype), "aqtx_fp_round: dtype must be bf16 or f32, got %d", p->dtype);
  const int cm = p->dtype == AQTX_BF16 ? 7 : 23;
  AQTX_REQUIRE(p->radix == 0 || p->radix == 2 || p->radix == 4, "aqtx_fp_round: radix must be 2 or 4, got %d", p->radix);
  const bool radix4 = p->radix == 4;
  AQTX_REQUIRE(!radix4 || p->dtype == AQTX_BF16, "aqtx_fp_round: radix 4 takes bf16 only");
  AQTX_REQUIRE(radix4 || (p->nexp >= 0 && p->nexp <= 7), "aqtx_fp_round: nexp %d outside 0..7", p->nexp);
  AQTX_REQUIRE(radix4 || (p->nmant >= 0 && p->nmant < cm),
               "aqtx_fp_round: nmant %d must be below the container's %d mantissa bits", p->nmant, cm);
  AQTX_REQUIRE(p->mode == AQTX_FP_NEAREST || p->mode == AQTX_FP_NOISE_JAX_BITS || p->mode == AQTX_FP_NOISE_INDEX,
               "aqtx_fp_round: unknown mode %d", p->mode);
  AQTX_REQUIRE(p->count >= 0, "aqtx_fp_round: negative count");
  AQTX_REQUIRE(p->mode != AQTX_FP_NOISE_INDEX || (p->noise_mod >= 1 && p->noise_mod <= 65536),
               "aqtx_fp_round: noise_mod must be in 1..65536");
  AQTX_REQUIRE(p->mode != AQTX_FP_NOISE_JAX_BITS || key_host != nullptr, "aqtx_fp_round: key is NULL");
  AQTX_REQUIRE(p->mode != AQTX_FP_NOISE_JAX_BITS || p->count < (int64_t)0xFFFFFFFFll,
               "aqtx_fp_round: count out of range for the random bit generator");
  if (p->count == 0) return 0;
  AQTX_REQUIRE(x != nullptr && out != nullptr, "aqtx_fp_round: NULL buffer");
  const size_t esize = dtype_size(p->dtype);
  AQTX_REQUIRE(((uintptr_t)x % esize) == 0 && ((uintptr_t)out % esize) == 0,
               "aqtx_fp_round: buffers must be aligned to the element size");

  FpArgs a{};
  a.x = x;
  a.out = out;
  a.count = p->count;
  a.noise_mod = p->mode == AQTX_FP_NOISE_INDEX ? p->noise_mod : 1;
  a.radix4 = radix4 ? 1 : 0;
  const int nmant = radix4 ? 0 : p->nmant, nexp = radix4 ? 3 : p->nexp;  // unread by the radix-4 branch
  a.trunc = (uint32_t)(cm - nmant);
  a.trunc_mask = (1u << a.trunc) - 1u;
  const uint32_t min_exp = 127u - (p->has_subnormals ? 1u : 0u);
  const uint32_t max_exp = min_exp + (1u << nexp) - 1u;
  const uint32_t mant_mask = (1u << cm) - 1u;
  a.min_repr = min_exp << cm;
  a.max_repr = (max_exp << cm) + (mant_mask & ~a.trunc_mask);
  a.nmant = nmant;
  a.sub = p->has_subnormals ? 1 : 0;
  a.nexp0 = nexp == 0;
  a.mode = p->mode;
  a.scale = (float)(1u << nmant);
  a.inv_scale = 1.0f / a.scale;
  a.max_sub = 1.0f - a.inv_scale;
  a.min_float = p->has_subnormals ? 0.5f : 1.0f;
  if (p->mode == AQTX_FP_NOISE_JAX_BITS) a.gen = make_bitgen(key_host, p->count, 16, p->partitionable);

  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool aligned = ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int vec = aligned ? (p->dtype == AQTX_BF16 ? 8 : 4) : 2;
  const int64_t blocks = (p->count + 256 * vec - 1) / (256 * vec);
  AQTX_REQUIRE(blocks < (1ll << 31), "aqtx_fp_round: count too large for one launch");
  if (p->mode == AQTX_FP_NOISE_JAX_BITS && !p->partitionable && aligned && (2 * (int64_t)a.gen.half) % vec == 0) {
    const int64_t pblocks = (2 * (int64_t)a.gen.half + 256 * vec - 1) / (256 * vec);
    if (p->dtype == AQTX_BF16) fp_round_paired_kernel<true, 8><<<(unsigned)pblocks, 256, 0, st>>>(a);
    else fp_round_paired_kernel<false, 4><<<(unsigned)pblocks, 256, 0, st>>>(a);
    AQTX_HIP_CHECK_LAUNCH("fp_round_paired_kernel");
    return 0;
  }
  if (p->dtype == AQTX_BF16) {
    if (aligned) fp_round_kernel<true, 8><<<(unsigned)blocks, 256, 0, st>>>(a);
    else fp_round_kernel<true, 2><<<(unsigned)blocks, 256, 0, st>>>(a);
  } else {
    if (aligned) fp_round_kernel<false, 4><<<(unsigned)blocks, 256, 0, st>>>(a);
    else fp_round_kernel<false, 2><<<(unsigned)blocks, 256, 0, st>>>(a);
  }
  AQTX_HIP_CHECK_LAUNCH("fp_round_kernel");
  return 0;
}

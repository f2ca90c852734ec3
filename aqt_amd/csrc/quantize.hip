// Abs-max calibration + quantization kernels (gfx950).
//
// One operand of the quantized dot_general goes through
//   scale = absmax / quant_bound            (calibration.py:117-157)
//   t     = x * (1 / scale)                 (aqt_tensor.py:125-159)
//   t     = t + noise; clip; round; cast    (int_numerics.py:81-111,
//                                            fp8_numerics.py:36-123)
// with every intermediate rounded to the dtype the reference holds it in.  Two
// launch shapes cover the layouts:
//   * "rows": the reduced axis is the contiguous one.  A segment (one row, or one
//     subchannel group of a row) is loaded once into registers by 16, 64 or 256
//     lanes, reduced with wavefront shuffles (+LDS across the four waves),
//     quantized from registers and stored: one HBM read, one write.
//   * "tile": the reduced axis is the strided one (or the whole tensor).  A
//     column abs-max pass (atomic max on the float bit pattern) is followed by a
//     128x64 tile pass that quantizes and, on request, writes the transposed
//     layout through LDS so that the consumer GEMM finds its contraction axis
//     contiguous.
#include "common.h"
#include <type_traits>

#include "threefry.h"

namespace aqtx {
namespace {

struct QArgs {
  const void* x;
  const float* prescale;
  void* q;
  float* scale;
  uint16_t* scale_bf16;  // optional second copy of the computed scales as bf16 elements
  uint32_t* ws_absmax;
  float* ws_inv;
  int64_t batch, rows, cols;
  int64_t L;        // rows kernel: segment length
  int64_t nseg;     // rows kernel: number of segments
  int64_t G;        // tile kernels: group length along rows
  int64_t ngroups;  // tile kernels: rows / G
  int64_t ssb, ssg, ssc;  // tile kernels: scale index strides
  int64_t nsb, nsr, nsc;  // noise counter strides
  int64_t psb;            // prescale batch stride
  float quant_bound, clip_bound;
  BitGen gen;
  const uint32_t* key_dev;  // optional: the two key words in device memory (replace gen.k0 / gen.k1)
  int noise;
  int ps_mode;
  int transpose_out;
  int out_dtype;
  int cbf;  // compute dtype is bf16
  int sbf;  // scale dtype is bf16
  int scale_given;
  int ws_zeroed;  // the abs-max words of the workspace are zero on entry
  int even_odd8;  // rows kernel: bytes of each group of 8 outputs stored as elements 0,2,4,6,1,3,5,7
  // Partial maxima of |q| along the axis that carries the scales, one byte per position of the reduced axis and
  // part (aqtx_quant_plan::other_axis_absmax): written by a launch (oa_out), or read in place of an abs-max pass
  // over this input (oa_in).
  uint8_t* oa_out;
  const uint8_t* oa_in;
  int64_t oa_in_parts;
};

// Kernel-side copy of the arguments with the PRNG key taken from device memory when the caller
// passed it there (a traced key under XLA, a key updated on the device between graph replays).
__device__ __forceinline__ QArgs with_device_key(const QArgs& in) {
  QArgs a = in;
  if (in.key_dev != nullptr) {
    a.gen.k0 = in.key_dev[0];
    a.gen.k1 = in.key_dev[1];
  }
  return a;
}

// The computed scale goes out as float32 and, when the caller keeps its scales in bf16, once
// more as bf16 elements (the value is already rounded to bf16, so the narrowing is exact).
__device__ __forceinline__ void store_scale(const QArgs& a, int64_t i, float v) {
  a.scale[i] = v;
  if (a.scale_bf16 != nullptr) a.scale_bf16[i] = (uint16_t)(__float_as_uint(v) >> 16);
}

// ---- typed vector loads ------------------------------------------------------
template <typename T> struct Loader;
template <> struct Loader<float> {
  static __device__ __forceinline__ void load8(const float* p, float* v) {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
};
template <> struct Loader<uint16_t> {  // bf16 bit patterns
  static __device__ __forceinline__ void load8(const uint16_t* p, float* v) {
    const uint4 a = *reinterpret_cast<const uint4*>(p);
    v[0] = __uint_as_float(a.x << 16); v[1] = __uint_as_float(a.x & 0xFFFF0000u);
    v[2] = __uint_as_float(a.y << 16); v[3] = __uint_as_float(a.y & 0xFFFF0000u);
    v[4] = __uint_as_float(a.z << 16); v[5] = __uint_as_float(a.z & 0xFFFF0000u);
    v[6] = __uint_as_float(a.w << 16); v[7] = __uint_as_float(a.w & 0xFFFF0000u);
  }
  static __device__ __forceinline__ float load1(const uint16_t* p) {
    return __uint_as_float(((uint32_t)*p) << 16);
  }
};
template <> struct Loader<int8_t> {
  static __device__ __forceinline__ void load8(const int8_t* p, float* v) {
    const uint2 a = *reinterpret_cast<const uint2*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[i] = (float)(int8_t)((a.x >> (8 * i)) & 0xFF);
      v[4 + i] = (float)(int8_t)((a.y >> (8 * i)) & 0xFF);
    }
  }
  static __device__ __forceinline__ float load1(const int8_t* p) { return (float)*p; }
};

__device__ __forceinline__ float rnd(float x, int bf) { return bf ? round_bf16(x) : x; }

// scale and reciprocal scale from the abs-max (calibration.py:145-157,
// aqt_tensor.py:151-155).
__device__ __forceinline__ void scale_from_absmax(float amax, const QArgs& a, float& scale,
                                                  float& inv) {
  if (amax == 0.0f) amax = 1.0f;
  float s = rnd(amax / a.quant_bound, a.cbf);
  s = rnd(s, a.sbf);
  float i = rnd(1.0f / s, a.sbf);
  if (isinf(i)) i = 1.0f;
  scale = s;
  inv = i;
}

__device__ __forceinline__ float inv_of_scale(float scale, const QArgs& a) {
  float i = rnd(1.0f / scale, a.sbf);
  if (isinf(i)) i = 1.0f;
  return i;
}

__device__ __forceinline__ float apply_prescale(float v, float ps, const QArgs& a) {
  // aqt_dot_general.py:714-720: lhs * scale_t.astype(lhs.dtype)
  return rnd(v * rnd(ps, a.cbf), a.cbf);
}

// The value after scaling, noise and clipping, still a float.
__device__ __forceinline__ float scaled_noisy_clipped(float v, float inv, uint64_t ctr,
                                                      const QArgs& a) {
  const int tbf = a.cbf & a.sbf;  // promote(x.dtype, scale.dtype)
  float t = rnd(v * inv, tbf);
  if (a.noise == AQTX_NOISE_JAX_UNIFORM) {
    const uint32_t bits = a.gen.draw(ctr);
    float u = __uint_as_float((bits >> 9) | 0x3F800000u) - 1.0f;
    u = fmaxf(0.0f, u);
    t = rnd(t + (u - 0.5f), tbf);
  } else if (a.noise == AQTX_NOISE_CUSTOM1) {
    const uint32_t bits = a.gen.draw(ctr);
    const float f = __uint_as_float((bits << 7) | 0x3F800000u);
    t = rnd(t + (f - 1.49999237060546875f), tbf);  // 1.5 - 2^-17
  } else if (a.noise == AQTX_NOISE_FP8_MANTISSA) {
    const int mant = (a.out_dtype == AQTX_E4M3) ? 3 : 2;
    const uint32_t bits = a.gen.draw(ctr);
    if (tbf) {
      const uint32_t mask = (1u << (7 - mant)) - 1u;
      uint32_t u = __float_as_uint(t) >> 16;
      u = ((u + (bits & mask)) & ~mask) & 0xFFFFu;
      t = __uint_as_float(u << 16);
    } else {
      const uint32_t mask = (1u << (23 - mant)) - 1u;
      uint32_t u = __float_as_uint(t);
      u = (u + (bits & mask)) & ~mask;
      t = __uint_as_float(u);
    }
  }
  t = fminf(fmaxf(t, -a.clip_bound), a.clip_bound);
  return t;
}

// float (already clipped) -> output byte
__device__ __forceinline__ uint32_t to_qbyte(float t, int out_dtype) {
  if (out_dtype == AQTX_E4M3) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(t, t, 0, false) & 0xFFu;
  } else if (out_dtype == AQTX_E5M2) {
    return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(t, t, 0, false) & 0xFFu;
  }
  return (uint32_t)((int)rintf(t)) & 0xFFu;
}

// ---- compile-time specialisations of the element pipeline ------------------------------
// SPEC 0: every flag is read from QArgs at run time (any dtype / numerics).
// SPEC 1: bf16 values, bf16 scale, integer out (int8, or int4 in an int8 byte), round to nearest
//         even (the forward operands).
// SPEC 3: bf16 values, bf16 scale, fp8 out (e4m3fn or e5m2), no noise.
// SPEC 5: SPEC 3 + fp8 mantissa stochastic rounding, 16-bit draws of the original layout.
// SPEC 2: SPEC 1 + jax.random.uniform noise in the original threefry counter layout (the
//         gradient-side operands).  With PAIR the two elements that share one threefry block
//         (indices i and i + total/2) are produced by the same thread from a single block.
template <int SPEC>
__device__ __forceinline__ float spec_scale(float v, float inv, const QArgs& a) {
  if constexpr (SPEC == 0) return rnd(v * inv, a.cbf & a.sbf);
  return round_bf16(v * inv);
}
__device__ __forceinline__ float uniform_noise(uint32_t bits) {
  // jax.random.uniform: f = bitcast(bits >> 9 | 0x3F800000) in [1, 2), u = f - 1, max(0, u); then
  // the centring of JaxUniform, u - 0.5.  f - 1 and u - 0.5 are exact (multiples of 2^-23 below 1)
  // and u >= 0, so the three steps equal the single exact subtraction f - 1.5.  The shift-and-or
  // is one funnel shift of {0x7F, bits} by 9.
  const uint32_t f = __builtin_amdgcn_alignbit(0x7Fu, bits, 9);
  return __uint_as_float(f) - 1.5f;
}
// Rounds two floats to bf16 (ties to even) in place with one packed conversion.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ void round_bf16_pair(float& a, float& b) {
  const bf16x2_t h = __builtin_convertvector(f32x2_t{a, b}, bf16x2_t);
  const uint32_t w = __builtin_bit_cast(uint32_t, h);
  a = __uint_as_float(w << 16);
  b = __uint_as_float(w & 0xFFFF0000u);
}
template <int SPEC>
__device__ __forceinline__ uint32_t spec_finish(float t, const QArgs& a) {
  // clip, round half to even, cast (int_numerics.py:99-110; fp8_numerics.py:112-123)
  if constexpr (SPEC == 0 || SPEC == 3 || SPEC == 5) {
    t = fminf(fmaxf(t, -a.clip_bound), a.clip_bound);
    return to_qbyte(t, a.out_dtype);
  }
  // clip in one median-of-three; round half to even and convert in one addition: after
  // t + 1.5 * 2^23 the low mantissa bits are the two's complement of the rounded integer
  // (|t| <= 127 here)
  t = __builtin_amdgcn_fmed3f(t, -a.clip_bound, a.clip_bound);
  return __float_as_uint(t + 12582912.0f) & 0xFFu;
}
// fp_mantissa_round on a bf16 value (fp8_numerics.py:36-64): add the masked random bits to the
// bit pattern, clear the low mantissa bits.
__device__ __forceinline__ float bf16_mantissa_sr(float t, uint32_t bits, uint32_t mask) {
  uint32_t u = __float_as_uint(t) >> 16;
  u = ((u + (bits & mask)) & ~mask) & 0xFFFFu;
  return __uint_as_float(u << 16);
}
// scale -> (noise) -> clip/round/cast for one element
template <int SPEC>
__device__ __forceinline__ uint32_t spec_quant(float v, float inv, uint64_t ctr, const QArgs& a) {
  if constexpr (SPEC == 0) {
    return to_qbyte(scaled_noisy_clipped(v, inv, ctr, a), a.out_dtype);
  } else {
    float t = spec_scale<SPEC>(v, inv, a);
    if constexpr (SPEC == 2) t = round_bf16(t + uniform_noise(a.gen.word_original((uint32_t)ctr)));
    if constexpr (SPEC == 5) {
      const uint32_t w = a.gen.word_original((uint32_t)(ctr >> 1));
      t = bf16_mantissa_sr(t, (ctr & 1) ? (w >> 16) : w, a.out_dtype == AQTX_E4M3 ? 0xFu : 0x1Fu);
    }
    return spec_finish<SPEC>(t, a);
  }
}
// The same for the noiseless integer pipelines (SPEC 0 with integer out, SPEC 1), which also hands out the clipped
// value before rounding: |q| = rint(|t|) and rint is monotonic, so a maximum of |q| can be kept as a maximum of
// |t| (one instruction per element) and rounded once at the end.
template <int SPEC>
__device__ __forceinline__ uint32_t spec_quant_mag(float v, float inv, uint64_t ctr, const QArgs& a, float& t_clipped) {
  static_assert(SPEC == 0 || SPEC == 1, "noiseless integer pipelines");
  if constexpr (SPEC == 0) {
    t_clipped = scaled_noisy_clipped(v, inv, ctr, a);
    return to_qbyte(t_clipped, a.out_dtype);
  } else {
    t_clipped = __builtin_amdgcn_fmed3f(spec_scale<1>(v, inv, a), -a.clip_bound, a.clip_bound);
    return __float_as_uint(t_clipped + 12582912.0f) & 0xFFu;
  }
}
// the pair (i, i + half) from one threefry block (SPEC 2, original layout, i < half)
__device__ __forceinline__ void pair_quant(float v0, float inv0, float v1, float inv1, uint32_t i,
                                           const QArgs& a, uint32_t& q0, uint32_t& q1) {
  const U2 bits = threefry2x32(a.gen.k0, a.gen.k1, i, i + a.gen.half);
  float t0 = v0 * inv0, t1 = v1 * inv1;
  round_bf16_pair(t0, t1);
  t0 += uniform_noise(bits.x);
  t1 += uniform_noise(bits.y);
  round_bf16_pair(t0, t1);
  q0 = spec_finish<2>(t0, a);
  q1 = spec_finish<2>(t1, a);
}
template <int SPEC>
__device__ __forceinline__ float spec_prescale(float v, float ps, const QArgs& a) {
  if constexpr (SPEC == 0) return apply_prescale(v, ps, a);
  return round_bf16(v * round_bf16(ps));
}
template <int SPEC>
__device__ __forceinline__ void spec_scale_from_absmax(float amax, const QArgs& a, float& scale, float& inv) {
  if constexpr (SPEC == 0) {
    scale_from_absmax(amax, a, scale, inv);
  } else {
    if (amax == 0.0f) amax = 1.0f;
    scale = round_bf16(amax / a.quant_bound);
    inv = round_bf16(1.0f / scale);
    if (isinf(inv)) inv = 1.0f;
  }
}

template <int LANES>
__device__ __forceinline__ float segment_max(float v, float* smem) {
  constexpr int W = LANES < 64 ? LANES : 64;
#pragma unroll
  for (int off = W / 2; off > 0; off >>= 1) v = nanmax(v, __shfl_xor(v, off, W));
  if constexpr (LANES >= 256) {  // the segment is the whole block
    const int wave = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) smem[wave] = v;
    __syncthreads();
    v = nanmax(nanmax(smem[0], smem[1]), nanmax(smem[2], smem[3]));
    if constexpr (LANES == 512) v = nanmax(v, nanmax(nanmax(smem[4], smem[5]), nanmax(smem[6], smem[7])));
  }
  return v;
}

// Eight row values kept in registers between the abs-max pass and the quantize pass.  bf16
// inputs of the specialised pipelines stay packed two per register (the prescaled value is
// rounded to bf16 as well), which halves the registers a row costs and doubles the waves per SIMD.
template <bool PACKED> struct RowVals;
template <> struct RowVals<false> {
  float f[8];
  __device__ __forceinline__ void put(const float* t) {
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = t[e];
  }
  __device__ __forceinline__ void get(float* t) const {
#pragma unroll
    for (int e = 0; e < 8; ++e) t[e] = f[e];
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int e = 0; e < 8; ++e) f[e] = 0.0f;
  }
};
template <> struct RowVals<true> {
  uint32_t w[4];
  __device__ __forceinline__ void put(const float* t) {  // t[e] are bf16-representable
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = __builtin_amdgcn_perm(__float_as_uint(t[2 * i + 1]), __float_as_uint(t[2 * i]), 0x07060302u);
  }
  __device__ __forceinline__ void get(float* t) const {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      t[2 * i] = __uint_as_float(w[i] << 16);
      t[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
  }
  __device__ __forceinline__ void zero() { w[0] = w[1] = w[2] = w[3] = 0u; }
};
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
// max of the two bf16 magnitudes of `w` against the running packed maxima: magnitudes of
// floats order like unsigned integers
__device__ __forceinline__ uint32_t packed_absmax(uint32_t m, uint32_t w) {
  const u16x2_t a = __builtin_bit_cast(u16x2_t, m), b = __builtin_bit_cast(u16x2_t, w & 0x7FFF7FFFu);
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
}

// Eight output bytes -> two words, in element order or as elements 0,2,4,6 | 1,3,5,7.
__device__ __forceinline__ uint2 pack8(const uint32_t (&q)[8], int even_odd8) {
  if (even_odd8)
    return make_uint2(q[0] | (q[2] << 8) | (q[4] << 16) | (q[6] << 24), q[1] | (q[3] << 8) | (q[5] << 16) | (q[7] << 24));
  return make_uint2(q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24), q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24));
}

// ---- rows kernel: reduced axis contiguous -------------------------------------
// PAIR (SPEC 2 only): the block owns segment s and segment s + nseg/2, whose elements share
// threefry blocks; requires whole rows as segments and the natural noise layout.
// A block is 256 threads, or 512 (LANES = 512: one long segment per block, half the row values per
// thread, so that six waves fit a SIMD: the stochastic pipeline is bound by vector instruction
// issue, and a wave issues one such instruction every ~12 cycles at best).
// COLMAX (whole rows as segments, one per block, no PAIR): the grid is smaller than the number of rows, a block
// walks rows blockIdx.x, + gridDim.x, ... and keeps, per column it owns, the largest |q| it wrote; at the end it
// stores them as row blockIdx.x of QArgs::oa_out ([gridDim.x][cols] bytes): what a later pass that calibrates the
// quantized values over the rows needs instead of reading them again.
template <typename TIn, int LANES, int ITERS, int SPEC, bool PAIR, bool COLMAX = false>
__global__ __launch_bounds__(LANES == 512 ? 512 : 256,
                             (COLMAX && ITERS <= 2 && SPEC != 0) ? 7 : LANES == 512 ? 3 : (sizeof(TIn) == 2 && SPEC != 0) ? 4 : 1)
void quant_rows_kernel(const QArgs a_in) {
  const QArgs a = with_device_key(a_in);
  constexpr int VEC = 8;
  constexpr int NT = LANES == 512 ? 512 : 256;
  constexpr int SEG_PER_BLOCK = NT / LANES;
  constexpr int NSET = PAIR ? 2 : 1;
  static_assert(!COLMAX || (!PAIR && SEG_PER_BLOCK == 1), "column maxima: one whole row per block");
  __shared__ float smem[NSET][NT / 64];
  const int tid = threadIdx.x;
  const int lane = tid % LANES;
  const int64_t nseg_grid = PAIR ? a.nseg / 2 : a.nseg;
  float colmax[COLMAX ? ITERS : 1][VEC];  // largest clipped |x / scale| per column (rounded at the end)
  if constexpr (COLMAX) {
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int e = 0; e < VEC; ++e) colmax[it][e] = 0.0f;
  }
  for (int64_t blk = blockIdx.x;; blk += gridDim.x) {
  if constexpr (COLMAX) {
    if (blk >= nseg_grid) break;  // uniform over the block
  }
  const int64_t seg0 = blk * SEG_PER_BLOCK + tid / LANES;
  const bool active = seg0 < nseg_grid;
  const int64_t segs_per_row = a.cols / a.L;

  constexpr bool PACKED = (sizeof(TIn) == 2) && (SPEC != 0);
  RowVals<PACKED> v[NSET][ITERS];
  float scale[NSET], inv[NSET];
  int64_t grow[NSET], col0[NSET];
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
    const int64_t seg = seg0 + (int64_t)s * nseg_grid;
    grow[s] = active ? seg / segs_per_row : 0;  // b * rows + r
    col0[s] = active ? (seg % segs_per_row) * a.L : 0;
    const int64_t b = grow[s] / a.rows, r = grow[s] % a.rows;
    const TIn* xp = reinterpret_cast<const TIn*>(a.x) + grow[s] * a.cols + col0[s];
    const float* psv = a.prescale + b * a.psb;
    float row_ps = 1.0f;
    if (a.ps_mode == AQTX_PRESCALE_PER_ROW) row_ps = psv[r];
    float amax = 0.0f;
    uint32_t amax_packed = 0u;
#pragma clang loop unroll(full)
    for (int it = 0; it < ITERS; ++it) {
      const int64_t j0 = (int64_t)(it * LANES + lane) * VEC;
      if (active && j0 < a.L) {
        bool stored = false;
        if constexpr (PACKED) {
          if (a.ps_mode == AQTX_PRESCALE_NONE) {  // the loaded words are the stored form
            const uint4 raw = *reinterpret_cast<const uint4*>(xp + j0);
            v[s][it].w[0] = raw.x; v[s][it].w[1] = raw.y; v[s][it].w[2] = raw.z; v[s][it].w[3] = raw.w;
#pragma unroll
            for (int i = 0; i < 4; ++i) amax_packed = packed_absmax(amax_packed, v[s][it].w[i]);
            stored = true;
          }
        }
        if (!stored) {
          float t[VEC];
          Loader<TIn>::load8(xp + j0, t);
          if (a.ps_mode == AQTX_PRESCALE_PER_ROW) {
#pragma unroll
            for (int e = 0; e < VEC; ++e) t[e] = spec_prescale<SPEC>(t[e], row_ps, a);
          } else if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
            const float4 p0 = *reinterpret_cast<const float4*>(psv + col0[s] + j0);
            const float4 p1 = *reinterpret_cast<const float4*>(psv + col0[s] + j0 + 4);
            const float ps[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
#pragma unroll
            for (int e = 0; e < VEC; ++e) t[e] = spec_prescale<SPEC>(t[e], ps[e], a);
          }
          v[s][it].put(t);
          if constexpr (PACKED) {  // the values are bf16 by now: two magnitudes per integer max
#pragma unroll
            for (int i = 0; i < 4; ++i) amax_packed = packed_absmax(amax_packed, v[s][it].w[i]);
          } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) amax = absmax_step(amax, t[e]);
          }
        }
      } else {
        v[s][it].zero();
      }
    }
    if constexpr (PACKED)
      amax = nanmax(amax, nanmax(__uint_as_float(amax_packed << 16), __uint_as_float(amax_packed & 0xFFFF0000u)));
    amax = segment_max<LANES>(amax, smem[s]);
    if (a.scale_given) {
      scale[s] = active ? a.scale[seg] : 1.0f;
      inv[s] = inv_of_scale(scale[s], a);
    } else {
      spec_scale_from_absmax<SPEC>(amax, a, scale[s], inv[s]);
      if (active && lane == 0) store_scale(a, seg, scale[s]);
    }
  }

  uint8_t* qp0 = reinterpret_cast<uint8_t*>(a.q) + grow[0] * a.cols + col0[0];
  if constexpr (PAIR) {
    uint8_t* qp1 = reinterpret_cast<uint8_t*>(a.q) + grow[1] * a.cols + col0[1];
    const uint32_t ctr_row = (uint32_t)(grow[0] * a.cols);  // natural layout: index of (row, 0)
#pragma clang loop unroll(full)
    for (int it = 0; it < ITERS; ++it) {
      const int64_t j0 = (int64_t)(it * LANES + lane) * VEC;
      if (active && j0 < a.L) {
        uint32_t q0[VEC], q1[VEC];
        float t0[VEC], t1[VEC];
        v[0][it].get(t0);
        v[1][it].get(t1);
#pragma unroll
        for (int e = 0; e < VEC; ++e)
          pair_quant(t0[e], inv[0], t1[e], inv[1], ctr_row + (uint32_t)(j0 + e), a, q0[e], q1[e]);
        *reinterpret_cast<uint2*>(qp0 + j0) = pack8(q0, a.even_odd8);
        *reinterpret_cast<uint2*>(qp1 + j0) = pack8(q1, a.even_odd8);
      }
    }
  } else {
    const int64_t b = grow[0] / a.rows, r = grow[0] % a.rows;
    const uint64_t ctr_row = (uint64_t)(b * a.nsb + r * a.nsr + col0[0] * a.nsc);
#pragma clang loop unroll(full)
    for (int it = 0; it < ITERS; ++it) {
      const int64_t j0 = (int64_t)(it * LANES + lane) * VEC;
      if (active && j0 < a.L) {
        uint32_t q[VEC];
        float t[VEC];
        v[0][it].get(t);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          if constexpr (COLMAX) {
            float tc;
            q[e] = spec_quant_mag<SPEC>(t[e], inv[0], ctr_row + (uint64_t)((j0 + e) * a.nsc), a, tc);
            colmax[it][e] = fmaxf(colmax[it][e], fabsf(tc));
          } else {
            q[e] = spec_quant<SPEC>(t[e], inv[0], ctr_row + (uint64_t)((j0 + e) * a.nsc), a);
          }
        }
        *reinterpret_cast<uint2*>(qp0 + j0) = pack8(q, a.even_odd8);
      }
    }
  }
  if constexpr (!COLMAX) break;
  __syncthreads();  // the next row's abs-max goes through the same LDS words
  }
  if constexpr (COLMAX) {
#pragma clang loop unroll(full)
    for (int it = 0; it < ITERS; ++it) {
      const int64_t j0 = (int64_t)(it * LANES + lane) * VEC;
      if (j0 < a.L) {
        uint32_t m[VEC];
#pragma unroll
        for (int e = 0; e < VEC; ++e) m[e] = (uint32_t)(int)rintf(colmax[it][e]);
        *reinterpret_cast<uint2*>(a.oa_out + (int64_t)blockIdx.x * a.cols + j0) = pack8(m, 0);
      }
    }
  }
}

// Generic rows kernel: any segment length / alignment; one wave per segment, two reads.
template <typename TIn>
__global__ __launch_bounds__(256) void quant_rows_generic_kernel(const QArgs a_in) {
  const QArgs a = with_device_key(a_in);
  const int lane = threadIdx.x & 63;
  const int64_t seg = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (seg >= a.nseg) return;  // the whole wave leaves together; no barrier below
  const int64_t segs_per_row = a.cols / a.L;
  const int64_t grow = seg / segs_per_row;
  const int64_t col0 = (seg % segs_per_row) * a.L;
  const int64_t b = grow / a.rows, r = grow % a.rows;
  const TIn* xp = reinterpret_cast<const TIn*>(a.x) + grow * a.cols + col0;
  auto value = [&](int64_t j) {
    float v = Loader<TIn>::load1(xp + j);
    if (a.ps_mode == AQTX_PRESCALE_PER_ROW) v = apply_prescale(v, a.prescale[b * a.psb + r], a);
    else if (a.ps_mode == AQTX_PRESCALE_PER_COL) v = apply_prescale(v, a.prescale[b * a.psb + col0 + j], a);
    return v;
  };
  float amax = 0.0f;
  for (int64_t j = lane; j < a.L; j += 64) amax = absmax_step(amax, value(j));
  amax = segment_max<64>(amax, nullptr);
  float scale, inv;
  if (a.scale_given) {
    scale = a.scale[seg];
    inv = inv_of_scale(scale, a);
  } else {
    scale_from_absmax(amax, a, scale, inv);
    if (lane == 0) store_scale(a, seg, scale);
  }
  uint8_t* qp = reinterpret_cast<uint8_t*>(a.q) + grow * a.cols + col0;
  const uint64_t ctr_row = (uint64_t)(b * a.nsb + r * a.nsr + col0 * a.nsc);
  for (int64_t j = lane; j < a.L; j += 64) {
    const float t = scaled_noisy_clipped(value(j), inv, ctr_row + (uint64_t)(j * a.nsc), a);
    qp[j] = (uint8_t)to_qbyte(t, a.out_dtype);
  }
}

// ---- tile kernels: reduced axis strided (or the whole tensor) -------------------

__global__ void fill_u32_kernel(uint32_t* p, int64_t n, uint32_t v) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}

constexpr int kAbsRowChunk = 64;

// Column abs-max: block = 4 waves x (64 lanes x VEC cols); the waves interleave
// over the rows of one chunk, partial maxima meet in LDS and leave through one
// atomic max per column (|x| >= 0, so the float bit pattern orders like a uint).
template <typename TIn, int VEC>
__global__ __launch_bounds__(256) void absmax_cols_kernel(const QArgs a) {
  __shared__ float smem[4][64 * VEC];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t c0 = ((int64_t)blockIdx.x * 64 + lane) * VEC;
  const int64_t chunks_per_group = (a.G + kAbsRowChunk - 1) / kAbsRowChunk;
  const int64_t g = blockIdx.y / chunks_per_group;
  const int64_t chunk = blockIdx.y % chunks_per_group;
  const int64_t b = blockIdx.z;
  const int64_t r_begin = g * a.G + chunk * kAbsRowChunk;
  int64_t r_end = r_begin + kAbsRowChunk;
  if (r_end > (g + 1) * a.G) r_end = (g + 1) * a.G;
  float m[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) m[e] = 0.0f;
  if (c0 < a.cols) {
    float ps[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) ps[e] = 1.0f;
    if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) ps[e] = a.prescale[b * a.psb + c0 + e];
    }
    const TIn* xb = reinterpret_cast<const TIn*>(a.x) + b * a.rows * a.cols + c0;
    for (int64_t r = r_begin + wave; r < r_end; r += 4) {
      float v[VEC];
      if constexpr (VEC == 8) Loader<TIn>::load8(xb + r * a.cols, v);
      else v[0] = Loader<TIn>::load1(xb + r * a.cols);
      if (a.ps_mode == AQTX_PRESCALE_PER_ROW) {
        const float rp = a.prescale[b * a.psb + r];
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = apply_prescale(v[e], rp, a);
      } else if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) v[e] = apply_prescale(v[e], ps[e], a);
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) m[e] = absmax_step(m[e], v[e]);
    }
  }
#pragma unroll
  for (int e = 0; e < VEC; ++e) smem[wave][lane * VEC + e] = m[e];
  __syncthreads();
  for (int i = threadIdx.x; i < 64 * VEC; i += 256) {
    const int64_t c = (int64_t)blockIdx.x * 64 * VEC + i;
    if (c < a.cols) {
      const float mm = nanmax(nanmax(smem[0][i], smem[1][i]), nanmax(smem[2][i], smem[3][i]));
      atomicMax(a.ws_absmax + b * a.ssb + g * a.ssg + c * a.ssc, __float_as_uint(mm));
    }
  }
}

// Whole-tensor abs-max per batch entry.
template <typename TIn>
__global__ __launch_bounds__(256) void absmax_all_kernel(const QArgs a) {
  __shared__ float smem[4];
  const int64_t b = blockIdx.y;
  const int64_t n = a.rows * a.cols;
  const TIn* xb = reinterpret_cast<const TIn*>(a.x) + b * n;
  float m = 0.0f;
  if (a.cols % 8 == 0 && (a.ps_mode != AQTX_PRESCALE_PER_COL || a.psb % 4 == 0)) {
    // 8 elements (one row segment) per lane and load
    const int64_t stride = (int64_t)gridDim.x * 256 * 8;
#pragma unroll 4
    for (int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8; i < n; i += stride) {
      float v[8];
      Loader<TIn>::load8(xb + i, v);
      if (a.ps_mode == AQTX_PRESCALE_PER_ROW) {
        const float rp = a.prescale[b * a.psb + i / a.cols];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = apply_prescale(v[e], rp, a);
      } else if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
        const float* pc = a.prescale + b * a.psb + i % a.cols;
        const float4 lo = *reinterpret_cast<const float4*>(pc), hi = *reinterpret_cast<const float4*>(pc + 4);
        const float ps[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = apply_prescale(v[e], ps[e], a);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) m = absmax_step(m, v[e]);
    }
  } else {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
      float v = Loader<TIn>::load1(xb + i);
      if (a.ps_mode == AQTX_PRESCALE_PER_ROW) v = apply_prescale(v, a.prescale[b * a.psb + i / a.cols], a);
      else if (a.ps_mode == AQTX_PRESCALE_PER_COL) v = apply_prescale(v, a.prescale[b * a.psb + i % a.cols], a);
      m = absmax_step(m, v);
    }
  }
  m = segment_max<256>(m, smem);
  if (threadIdx.x == 0) atomicMax(a.ws_absmax + b * a.ssb, __float_as_uint(m));
}

// abs-max bit patterns -> scale (output) and reciprocal scale (workspace).
__global__ void finalize_scales_kernel(const QArgs a, int64_t n) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float scale, inv;
  if (a.scale_given) {
    scale = a.scale[i];
    inv = inv_of_scale(scale, a);
  } else {
    scale_from_absmax(__uint_as_float(a.ws_absmax[i]), a, scale, inv);
    a.ws_absmax[i] = 0u;  // the abs-max words leave as they have to arrive: zero
    store_scale(a, i, scale);
  }
  a.ws_inv[i] = inv;
}

// Partial maxima of |x| (bytes, [parts][n], written by an earlier launch next to the int8 values this one reads)
// -> scale (output) and reciprocal scale (workspace), in place of the abs-max pass and finalize_scales_kernel.
// A block takes 16 scales: thread t folds the 16 bytes of parts t, t + 256, ... (as eight pairs of 16-bit lanes,
// two maxima per instruction), the threads meet through wave shuffles and LDS.  (64 scales per block, whose loads
// use whole 64-byte sectors, leave 64 blocks for 4096 scales and measured slower: 11.6 against 8.1 us on average
// over 1792 and 224 parts.)
typedef unsigned short u16x2_max_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pk_max_u16(uint32_t x, uint32_t y) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(u16x2_max_t, x),
                                                                __builtin_bit_cast(u16x2_max_t, y)));
}
__global__ __launch_bounds__(256) void finalize_partials_kernel(const QArgs a, int64_t n) {
  __shared__ uint32_t smax[4][8];
  const int64_t c0 = (int64_t)blockIdx.x * 16;  // n is a multiple of 16 here
  uint32_t m[8];  // m[2 i] = bytes 0 and 2 of word i in 16-bit lanes, m[2 i + 1] = bytes 1 and 3
#pragma unroll
  for (int i = 0; i < 8; ++i) m[i] = 0u;
  for (int64_t p = threadIdx.x; p < a.oa_in_parts; p += 256) {
    const uint4 w = *reinterpret_cast<const uint4*>(a.oa_in + p * n + c0);
    const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      m[2 * i] = pk_max_u16(m[2 * i], ww[i] & 0x00FF00FFu);
      m[2 * i + 1] = pk_max_u16(m[2 * i + 1], (ww[i] >> 8) & 0x00FF00FFu);
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) m[i] = pk_max_u16(m[i], (uint32_t)__shfl_xor((int)m[i], off, 64));
  }
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) {
#pragma unroll
    for (int i = 0; i < 8; ++i) smax[wave][i] = m[i];
  }
  __syncthreads();
  if (threadIdx.x < 16) {
    // column c0 + t is byte t % 4 of word t / 4: lane (t % 4) / 2 of m[2 (t / 4) + t % 2]
    const int t = threadIdx.x, i = 2 * (t >> 2) + (t & 1), hi = (t >> 1) & 1;
    uint32_t v = pk_max_u16(pk_max_u16(smax[0][i], smax[1][i]), pk_max_u16(smax[2][i], smax[3][i]));
    v = hi ? v >> 16 : v & 0xFFFFu;
    float scale, inv;
    scale_from_absmax((float)v, a, scale, inv);
    store_scale(a, c0 + t, scale);
    a.ws_inv[c0 + t] = inv;
  }
}

constexpr int kTileR = 128, kTileC = 64, kTilePad = 132;

// 128x64 tile: thread (rg = tid/8, cc = tid%8) owns rows 4*rg..+3, cols 8*cc..+7.
// PAIR (SPEC 2, and SPEC 5 with value 1): 1 = the block also owns the tile `rows/2` further down (natural noise
// layout), 2 = the tile `cols/2` further right (noise counters of the transposed tensor); the
// two tiles' elements share threefry blocks.
// ROWMAX (no PAIR; every tile interior): the block also finds, for each of its 128 rows, the largest |q| among its 64
// columns, and stores them as bytes rows r0.. of row blockIdx.x of QArgs::oa_out ([column tiles][rows]).
template <typename TIn, int SPEC, int PAIR, bool ROWMAX = false>
__global__ __launch_bounds__(256) void quant_tile_kernel(const QArgs a_in) {
  static_assert(!ROWMAX || PAIR == 0, "row maxima: one tile per block");
  const QArgs a = with_device_key(a_in);
  constexpr int NSET = PAIR ? 2 : 1;
  __shared__ uint32_t lds[NSET][kTileC * kTilePad / 4];
  const int tid = threadIdx.x;
  const int cc = tid & 7, rg = tid >> 3;
  const int64_t b = blockIdx.z;
  const TIn* xb = reinterpret_cast<const TIn*>(a.x) + b * a.rows * a.cols;
  uint8_t* qb = reinterpret_cast<uint8_t*>(a.q) + b * a.rows * a.cols;
  const bool vec_ok = (a.cols % 8) == 0;
  int64_t r0[NSET], c0[NSET];
  r0[0] = (int64_t)blockIdx.y * kTileR;
  c0[0] = (int64_t)blockIdx.x * kTileC;
  // the first tile of a pair stays inside the first half of the paired axis
  const int64_t row_lim = PAIR == 1 ? a.rows / 2 : a.rows;
  const int64_t col_lim = PAIR == 2 ? a.cols / 2 : a.cols;
  if constexpr (PAIR == 1) { r0[1] = r0[0] + a.rows / 2; c0[1] = c0[0]; }
  if constexpr (PAIR == 2) { r0[1] = r0[0]; c0[1] = c0[0] + a.cols / 2; }

  uint32_t packed[NSET][8];  // packed[s][e] = bytes of rows 4*rg..4*rg+3 at col c+e
#pragma unroll
  for (int s = 0; s < NSET; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) packed[s][e] = 0u;

  // Tiles that lie wholly inside the tensor (and inside the first half of a paired axis) take a
  // branch-free path with vector loads of the reciprocal scales and the pre-scale factors.
  const bool interior = vec_ok && (r0[0] + kTileR <= row_lim) && (c0[0] + kTileC <= col_lim) &&
                        (a.ssc == 0 || (a.ssc == 1 && a.ssb % 4 == 0 && a.ssg % 4 == 0 &&
                                        ((uintptr_t)a.ws_inv % 16) == 0)) &&
                        (a.ps_mode != AQTX_PRESCALE_PER_COL || a.psb % 4 == 0);
  auto load8f = [](const float* p, float* v) {
    const float4 lo = *reinterpret_cast<const float4*>(p), hi = *reinterpret_cast<const float4*>(p + 4);
    v[0] = lo.x; v[1] = lo.y; v[2] = lo.z; v[3] = lo.w; v[4] = hi.x; v[5] = hi.y; v[6] = hi.z; v[7] = hi.w;
  };
  uint32_t rowmax = 0u;  // ROWMAX: byte j = largest |q| of row r0 + 4 * rg + j among the tile's 64 columns
  auto rows = [&](auto fast_tag) {
    constexpr bool FAST = decltype(fast_tag)::value;
    float ps_col[NSET][8];
    if constexpr (FAST) {
      if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
#pragma unroll
        for (int s = 0; s < NSET; ++s) load8f(a.prescale + b * a.psb + c0[s] + cc * 8, ps_col[s]);
      }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int64_t rl = r0[0] + rg * 4 + j;  // position inside the first tile's half
      const int64_t cl = c0[0] + cc * 8;
      if (FAST || (rl < row_lim && cl < col_lim)) {
        const int nvalid = FAST ? 8 : ((col_lim - cl) >= 8 ? 8 : (int)(col_lim - cl));
        float x[NSET][8], inv[NSET][8];
#pragma unroll
        for (int s = 0; s < NSET; ++s) {
          const int64_t r = r0[s] + rg * 4 + j, c = c0[s] + cc * 8;
          if (FAST || vec_ok) {
            Loader<TIn>::load8(xb + r * a.cols + c, x[s]);
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
              x[s][e] = e < nvalid ? Loader<TIn>::load1(xb + r * a.cols + c + e) : 0.0f;
          }
          const int64_t sbase = b * a.ssb + (r / a.G) * a.ssg;
          if (a.ps_mode == AQTX_PRESCALE_PER_ROW) {
            const float rp = a.prescale[b * a.psb + r];
#pragma unroll
            for (int e = 0; e < 8; ++e) x[s][e] = spec_prescale<SPEC>(x[s][e], rp, a);
          } else if (a.ps_mode == AQTX_PRESCALE_PER_COL) {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              if constexpr (FAST) x[s][e] = spec_prescale<SPEC>(x[s][e], ps_col[s][e], a);
              else if (e < nvalid) x[s][e] = spec_prescale<SPEC>(x[s][e], a.prescale[b * a.psb + c + e], a);
            }
          }
          if constexpr (FAST) {
            if (a.ssc == 0) {
              const float v = a.ws_inv[sbase];
#pragma unroll
              for (int e = 0; e < 8; ++e) inv[s][e] = v;
            } else {
              load8f(a.ws_inv + sbase + c, inv[s]);
            }
          } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) inv[s][e] = e < nvalid ? a.ws_inv[sbase + (c + e) * a.ssc] : 1.0f;
          }
        }
        uint32_t w[NSET][2];
#pragma unroll
        for (int s = 0; s < NSET; ++s) w[s][0] = w[s][1] = 0u;
        U2 wbits{0u, 0u};  // SPEC 5: the 32-bit word(s) two neighbouring elements draw their 16 bits from
        float rm = 0.0f;   // ROWMAX: largest clipped |x / scale| of this row among this thread's 8 columns
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          if (FAST || e < nvalid) {
            uint32_t qv[NSET];
            if constexpr (SPEC == 5) {
              // 16-bit draws: elements 2w and 2w+1 share word w; with PAIR the block (w, w + half)
              // also serves the same two elements of the tile rows/2 further down.
              const uint32_t sr_mask = a.out_dtype == AQTX_E4M3 ? 0xFu : 0x1Fu;
              const uint64_t ctr = (uint64_t)(b * a.nsb + rl * a.nsr + (cl + e) * a.nsc);
              if ((e & 1) == 0) {
                if constexpr (PAIR) {
                  wbits = threefry2x32(a.gen.k0, a.gen.k1, (uint32_t)(ctr >> 1), (uint32_t)(ctr >> 1) + a.gen.half);
                } else {
                  wbits.x = a.gen.word_original((uint32_t)(ctr >> 1));
                }
              }
              const int sh = (e & 1) * 16;
#pragma unroll
              for (int s = 0; s < NSET; ++s) {
                float t = round_bf16(x[s][e] * inv[s][e]);
                t = bf16_mantissa_sr(t, (s == 0 ? wbits.x : wbits.y) >> sh, sr_mask);
                qv[s] = spec_finish<5>(t, a);
              }
            } else if constexpr (PAIR) {
              const uint32_t i = (uint32_t)((r0[0] + rg * 4 + j) * a.nsr + (c0[0] + cc * 8 + e) * a.nsc);
              pair_quant(x[0][e], inv[0][e], x[1][e], inv[1][e], i, a, qv[0], qv[1]);
            } else if constexpr (ROWMAX) {
              float tc;
              qv[0] = spec_quant_mag<SPEC>(x[0][e], inv[0][e], 0, a, tc);
              rm = fmaxf(rm, fabsf(tc));
            } else {
              const uint64_t ctr = (uint64_t)(b * a.nsb + rl * a.nsr + (cl + e) * a.nsc);
              qv[0] = spec_quant<SPEC>(x[0][e], inv[0][e], ctr, a);
            }
#pragma unroll
            for (int s = 0; s < NSET; ++s) {
              w[s][e >> 2] |= qv[s] << (8 * (e & 3));
              packed[s][e] |= qv[s] << (8 * j);
            }
          }
        }
        if constexpr (ROWMAX) {
          // every tile is interior here, so all lanes are in this branch: the 8 threads of a row (consecutive lanes)
          // meet by shuffles; rint(max |t|) = max |q|
#pragma unroll
          for (int off = 1; off < 8; off <<= 1) rm = fmaxf(rm, __shfl_xor(rm, off, 64));
          rowmax |= (uint32_t)(int)rintf(rm) << (8 * j);
        }
        if (!a.transpose_out) {
#pragma unroll
          for (int s = 0; s < NSET; ++s) {
            const int64_t r = r0[s] + rg * 4 + j, c = c0[s] + cc * 8;
            if (FAST || vec_ok) {
              *reinterpret_cast<uint2*>(qb + r * a.cols + c) = make_uint2(w[s][0], w[s][1]);
            } else {
              for (int e = 0; e < nvalid; ++e)
                qb[r * a.cols + c + e] = (uint8_t)(w[s][e >> 2] >> (8 * (e & 3)));
            }
          }
        }
      }
    }
  };
  if (interior) rows(std::true_type{});
  else rows(std::false_type{});
  if constexpr (ROWMAX) {
    if (cc == 0)
      *reinterpret_cast<uint32_t*>(a.oa_out + ((int64_t)blockIdx.x * a.rows + r0[0] + rg * 4)) = rowmax;
  }
  if (!a.transpose_out) return;  // uniform across the block

  // Transposed write: LDS holds each tile as [col][row bytes], row stride 132 B.
#pragma unroll
  for (int s = 0; s < NSET; ++s)
#pragma unroll
    for (int e = 0; e < 8; ++e) lds[s][((cc * 8 + e) * kTilePad + rg * 4) / 4] = packed[s][e];
  __syncthreads();
  // thread -> (col = tid/8 + 32*h, 16-byte chunk = tid%8) of the [64][128] byte tile
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int col = (tid >> 3) + 32 * h;
      const int chunk = tid & 7;
      const int64_t gc_l = c0[0] + col, gr_l = r0[0] + chunk * 16;  // bounds in first-tile terms
      const int64_t gc = c0[s] + col, gr = r0[s] + chunk * 16;
      if (gc_l < col_lim && gr_l < row_lim) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) w[i] = lds[s][(col * kTilePad + chunk * 16) / 4 + i];
        uint8_t* dst = qb + gc * a.rows + gr;
        const int64_t lim = row_lim - gr_l;
        if ((a.rows % 16) == 0 && (PAIR != 1 || ((a.rows / 2) % 16) == 0)) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(w[0], w[1], w[2], w[3]);
        } else {
          const int nv = lim >= 16 ? 16 : (int)lim;
          for (int i = 0; i < nv; ++i) dst[i] = (uint8_t)(w[i >> 2] >> (8 * (i & 3)));
        }
      }
    }
  }
}

__global__ void random_bits_kernel(BitGen gen, int64_t n, void* out) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t v = gen.draw((uint64_t)i);
  if (gen.width == 16) reinterpret_cast<uint16_t*>(out)[i] = (uint16_t)v;
  else reinterpret_cast<uint32_t*>(out)[i] = v;
}

// out[b, r, c] = cast(q) * scale (aqt_tensor.py:179-183), one thread per element.
template <typename TOut>
__global__ void dequant_kernel(const QArgs a, int fp8_kind) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t per_b = a.rows * a.cols;
  if (i >= a.batch * per_b) return;
  const int64_t b = i / per_b, rc = i % per_b, r = rc / a.cols, c = rc % a.cols;
  const uint8_t* qb = reinterpret_cast<const uint8_t*>(a.x) + b * per_b;
  const uint8_t raw = a.transpose_out ? qb[c * a.rows + r] : qb[rc];
  float v;
  if (fp8_kind == AQTX_E4M3) v = __builtin_amdgcn_cvt_f32_fp8((int)raw, 0);
  else if (fp8_kind == AQTX_E5M2) v = __builtin_amdgcn_cvt_f32_bf8((int)raw, 0);
  else v = (float)(int8_t)raw;
  const float s = a.scale[b * a.ssb + (r / a.G) * a.ssg + (c / a.L) * a.ssc];
  v = rnd(v, a.cbf);
  v = rnd(v * s, a.cbf & a.sbf);
  v = rnd(v, a.cbf);
  if constexpr (sizeof(TOut) == 2) reinterpret_cast<uint16_t*>(a.q)[i] = bf16_bits(v);
  else reinterpret_cast<float*>(a.q)[i] = v;
}

// ---- host side ---------------------------------------------------------------------

int validate(const aqtx_quant_plan* p) {
  AQTX_REQUIRE(p != nullptr, "aqtx_quantize: plan is NULL");
  AQTX_REQUIRE(p->in_dtype == AQTX_F32 || p->in_dtype == AQTX_BF16 || p->in_dtype == AQTX_I8,
               "aqtx_quantize: unsupported in_dtype %d", p->in_dtype);
  AQTX_REQUIRE(is_float_dtype(p->compute_dtype),
               "aqtx_quantize: compute_dtype must be f32 or bf16, got %d", p->compute_dtype);
  AQTX_REQUIRE(p->in_dtype == AQTX_I8 || p->in_dtype == p->compute_dtype,
               "aqtx_quantize: float input must be held in compute_dtype (in %d, compute %d)",
               p->in_dtype, p->compute_dtype);
  AQTX_REQUIRE(is_float_dtype(p->scale_dtype),
               "aqtx_quantize: scale_dtype must be f32 or bf16, got %d", p->scale_dtype);
  AQTX_REQUIRE(p->out_dtype == AQTX_I8 || p->out_dtype == AQTX_I4 || p->out_dtype == AQTX_E4M3 ||
                   p->out_dtype == AQTX_E5M2,
               "aqtx_quantize: unsupported out_dtype %d", p->out_dtype);
  AQTX_REQUIRE(p->batch >= 0 && p->rows >= 0 && p->cols >= 0, "aqtx_quantize: negative shape");
  AQTX_REQUIRE(p->reduce >= AQTX_REDUCE_COLS && p->reduce <= AQTX_REDUCE_ALL_BATCH,
               "aqtx_quantize: unknown reduce mode %d", p->reduce);
  AQTX_REQUIRE(p->group >= 0, "aqtx_quantize: negative group");
  if (p->group > 0) {
    AQTX_REQUIRE(p->reduce == AQTX_REDUCE_COLS || p->reduce == AQTX_REDUCE_ROWS,
                 "aqtx_quantize: group needs REDUCE_COLS or REDUCE_ROWS");
    const int64_t axis = p->reduce == AQTX_REDUCE_COLS ? p->cols : p->rows;
    AQTX_REQUIRE(axis % p->group == 0,
                 "aqtx_quantize: group %lld does not divide the reduced axis %lld",
                 (long long)p->group, (long long)axis);
  }
  AQTX_REQUIRE(!(p->transpose_out && p->reduce == AQTX_REDUCE_COLS),
               "aqtx_quantize: transpose_out is not supported with REDUCE_COLS");
  AQTX_REQUIRE(p->noise >= AQTX_NOISE_NONE && p->noise <= AQTX_NOISE_FP8_MANTISSA,
               "aqtx_quantize: unknown noise kind %d", p->noise);
  const bool fp8 = p->out_dtype == AQTX_E4M3 || p->out_dtype == AQTX_E5M2;
  AQTX_REQUIRE(!(p->noise == AQTX_NOISE_FP8_MANTISSA && !fp8),
               "aqtx_quantize: mantissa noise needs an fp8 out_dtype");
  AQTX_REQUIRE(!((p->noise == AQTX_NOISE_JAX_UNIFORM || p->noise == AQTX_NOISE_CUSTOM1) && fp8),
               "aqtx_quantize: additive noise needs an integer out_dtype");
  if (p->noise != AQTX_NOISE_NONE) {
    AQTX_REQUIRE(p->noise_total > 0 && p->noise_total < (int64_t)0xFFFFFFFFll,
                 "aqtx_quantize: noise_total %lld out of range (1 .. 2^32-2)",
                 (long long)p->noise_total);
  }
  AQTX_REQUIRE(p->prescale >= AQTX_PRESCALE_NONE && p->prescale <= AQTX_PRESCALE_PER_COL,
               "aqtx_quantize: unknown prescale mode %d", p->prescale);
  AQTX_REQUIRE(p->quant_bound > 0.0f && p->clip_bound > 0.0f,
               "aqtx_quantize: bounds must be positive");
  return 0;
}

int64_t scale_count(const aqtx_quant_plan* p) {
  switch (p->reduce) {
    case AQTX_REDUCE_COLS: return p->batch * p->rows * (p->group ? p->cols / p->group : 1);
    case AQTX_REDUCE_ROWS: return p->batch * (p->group ? p->rows / p->group : 1) * p->cols;
    case AQTX_REDUCE_ALL: return p->batch;
    default: return 1;
  }
}

int noise_width(const aqtx_quant_plan* p) {
  if (p->noise == AQTX_NOISE_CUSTOM1) return 16;
  if (p->noise == AQTX_NOISE_FP8_MANTISSA)
    return (p->compute_dtype == AQTX_BF16 && p->scale_dtype == AQTX_BF16) ? 16 : 32;
  return 32;
}

// Which compile-time specialisation (see spec_quant) serves this plan.
int spec_of(const QArgs& a, int partitionable) {
  if (a.cbf && a.sbf && (a.out_dtype == AQTX_E4M3 || a.out_dtype == AQTX_E5M2)) {
    if (a.noise == AQTX_NOISE_NONE) return 3;
    if (a.noise == AQTX_NOISE_FP8_MANTISSA && !partitionable && a.gen.width == 16 && a.nsc == 1 &&
        a.nsr % 2 == 0 && a.nsb % 2 == 0)
      return 5;  // neighbouring elements draw from one word, starting at an even counter
    return 0;
  }
  if (!(a.cbf && a.sbf && (a.out_dtype == AQTX_I8 || a.out_dtype == AQTX_I4))) return 0;
  if (a.noise == AQTX_NOISE_NONE) return 1;
  if (a.noise == AQTX_NOISE_JAX_UNIFORM && !partitionable) return 2;
  return 0;
}

// Blocks of the row kernel that also writes column maxima, each walking rows: seven per CU of the largest part, as
// many as its registers (67 with 16 running maxima) let a CU hold (measured on 8192 rows of 4096 bf16 values, 21 us
// without the maxima: 62 us with 256 blocks, 40 with 512, 30 with 1024).
constexpr int64_t kColmaxBlocks = 7 * 256;

// Whether the row kernels can leave column maxima of |q| behind for this plan: whole rows of 520 to 8192
// aligned values as segments, one batch entry, integer values rounded to nearest.
bool rows_colmax_ok(const aqtx_quant_plan* p) {
  return p->reduce == AQTX_REDUCE_COLS && p->batch == 1 && p->group == 0 && !p->transpose_out &&
         p->noise == AQTX_NOISE_NONE && (p->out_dtype == AQTX_I8 || p->out_dtype == AQTX_I4) &&
         p->out_k_order == AQTX_K_NATURAL && p->cols % 8 == 0 && p->cols > 512 && p->cols <= 8192 && p->rows > 0;
}

template <typename TIn, int SPEC>
int launch_rows_colmax(const QArgs& a, hipStream_t st) {
  const int64_t L = a.L;
  const int64_t blocks = a.nseg < kColmaxBlocks ? a.nseg : kColmaxBlocks;  // = aqtx_quantize_other_axis_parts: rows of oa_out
#define AQTX_ROWS_CM(ITERS)                                                                                  \
  {                                                                                                          \
    quant_rows_kernel<TIn, 256, ITERS, SPEC, false, true><<<dim3((unsigned)blocks), 256, 0, st>>>(a);        \
    AQTX_HIP_CHECK_LAUNCH("quant_rows_kernel, column maxima");                                               \
    return 0;                                                                                                \
  }
  if (L <= 2048) AQTX_ROWS_CM(1)
  if (L <= 4096) AQTX_ROWS_CM(2)
  AQTX_ROWS_CM(4)
#undef AQTX_ROWS_CM
}

template <typename TIn, int SPEC, bool PAIR>
int launch_rows_spec(const QArgs& a, hipStream_t st) {
  const int64_t L = a.L;
  const int64_t nseg = PAIR ? a.nseg / 2 : a.nseg;
#define AQTX_ROWS(LANES, ITERS)                                                        \
  {                                                                                    \
    constexpr int kThreads = LANES == 512 ? 512 : 256;                                 \
    const int64_t blocks = (nseg + (kThreads / LANES) - 1) / (kThreads / LANES);       \
    quant_rows_kernel<TIn, LANES, ITERS, SPEC, PAIR><<<dim3((unsigned)blocks), kThreads, 0, st>>>(a); \
    AQTX_HIP_CHECK_LAUNCH("quant_rows_kernel");                                        \
    return 0;                                                                          \
  }
  if (L <= 128) AQTX_ROWS(16, 1)
  if (L <= 512) AQTX_ROWS(64, 1)
  if (L <= 2048) AQTX_ROWS(256, 1)
  if (L <= 4096) AQTX_ROWS(256, 2)
  if (L <= 8192) AQTX_ROWS(256, 4)
  if (SPEC == 2 && sizeof(TIn) == 2) AQTX_ROWS(512, 4)
  AQTX_ROWS(256, 8)
#undef AQTX_ROWS
}

template <typename TIn>
int launch_rows(const QArgs& a, int partitionable, hipStream_t st) {
  const int64_t L = a.L;
  const bool aligned = (L % 8 == 0) && (a.cols % 8 == 0);
  if (!aligned || L > 16384) {
    AQTX_REQUIRE(!a.even_odd8, "aqtx_quantize: out_k_order = EVEN_ODD8 needs cols and group to be multiples of 8 and "
                 "segments of at most 16384");
    const int64_t blocks = (a.nseg + 3) / 4;
    quant_rows_generic_kernel<TIn><<<dim3((unsigned)blocks), 256, 0, st>>>(a);
    AQTX_HIP_CHECK_LAUNCH("quant_rows_generic_kernel");
    return 0;
  }
  const int spec = spec_of(a, partitionable);
  if (a.oa_out != nullptr) {  // (the caller has checked rows_colmax_ok: noise none, so spec is 1 or 0)
    if (spec == 1) return launch_rows_colmax<TIn, 1>(a, st);
    return launch_rows_colmax<TIn, 0>(a, st);
  }
  if (spec == 1) return launch_rows_spec<TIn, 1, false>(a, st);
  if (spec == 3) return launch_rows_spec<TIn, 3, false>(a, st);
  if (spec == 5) return launch_rows_spec<TIn, 5, false>(a, st);
  if (spec == 2) {
    // one threefry block serves elements i and i + total/2: pair whole rows when the noise
    // counters follow the natural [batch*rows, cols] order
    const bool natural = a.nsc == 1 && a.nsr == a.cols && (a.batch == 1 || a.nsb == a.rows * a.cols) &&
                         L == a.cols && (a.nseg % 2 == 0);
    if (natural) return launch_rows_spec<TIn, 2, true>(a, st);
    return launch_rows_spec<TIn, 2, false>(a, st);
  }
  return launch_rows_spec<TIn, 0, false>(a, st);
}

// Whether the tile kernel can leave row maxima of |q| behind for this plan: one scale per column over whole
// columns, every 128 x 64 tile inside the tensor, one batch entry, integer values rounded to nearest.
bool tiles_rowmax_ok(const aqtx_quant_plan* p) {
  return p->reduce == AQTX_REDUCE_ROWS && p->batch == 1 && p->group == 0 && p->noise == AQTX_NOISE_NONE &&
         (p->out_dtype == AQTX_I8 || p->out_dtype == AQTX_I4) && p->rows > 0 && p->cols > 0 &&
         p->rows % kTileR == 0 && p->cols % kTileC == 0;
}

template <typename TIn>
int launch_tiles(const QArgs& a, int reduce, int partitionable, int64_t nscales, hipStream_t st) {
  if (a.oa_in != nullptr) {
    finalize_partials_kernel<<<dim3((unsigned)(nscales / 16)), 256, 0, st>>>(a, nscales);
    AQTX_HIP_CHECK_LAUNCH("finalize_partials_kernel");
  } else {
  if (!a.scale_given) {
    if (!a.ws_zeroed) {
      fill_u32_kernel<<<dim3((unsigned)((nscales + 255) / 256)), 256, 0, st>>>(a.ws_absmax, nscales, 0u);
      AQTX_HIP_CHECK_LAUNCH("fill_u32_kernel");
    }
    if (reduce == AQTX_REDUCE_ALL || reduce == AQTX_REDUCE_ALL_BATCH) {
      int64_t nblk = (a.rows * a.cols + 256 * 16 - 1) / (256 * 16);
      // Every block ends in one atomic max.  Atomics on one address take turns (about 10 ns each,
      // measured), and so do those on the neighbouring words of the batch entries, which share a
      // cache line: 32 entries x 98 blocks took 31 us for 26 MB.  So the launch as a whole gets at
      // most one block per 48 KiB of input (the time to stream that much), between 256 and 2048.
      const int64_t total_bytes = a.batch * a.rows * a.cols * (int64_t)sizeof(TIn);
      int64_t cap_total = total_bytes / (48 << 10);
      cap_total = cap_total < 256 ? 256 : cap_total > 2048 ? 2048 : cap_total;
      const int64_t cap = a.batch >= cap_total ? 1 : cap_total / a.batch;
      if (nblk > cap) nblk = cap;
      if (nblk < 1) nblk = 1;
      absmax_all_kernel<TIn><<<dim3((unsigned)nblk, (unsigned)a.batch), 256, 0, st>>>(a);
      AQTX_HIP_CHECK_LAUNCH("absmax_all_kernel");
    } else {
      const int64_t chunks = a.ngroups * ((a.G + kAbsRowChunk - 1) / kAbsRowChunk);
      if (a.cols % 8 == 0) {
        dim3 grid((unsigned)((a.cols + 511) / 512), (unsigned)chunks, (unsigned)a.batch);
        absmax_cols_kernel<TIn, 8><<<grid, 256, 0, st>>>(a);
      } else {
        dim3 grid((unsigned)((a.cols + 63) / 64), (unsigned)chunks, (unsigned)a.batch);
        absmax_cols_kernel<TIn, 1><<<grid, 256, 0, st>>>(a);
      }
      AQTX_HIP_CHECK_LAUNCH("absmax_cols_kernel");
    }
  }
  finalize_scales_kernel<<<dim3((unsigned)((nscales + 255) / 256)), 256, 0, st>>>(a, nscales);
  AQTX_HIP_CHECK_LAUNCH("finalize_scales_kernel");
  }
  const int spec = spec_of(a, partitionable);
  auto grid_for = [&](int pair) {
    const int64_t rows = pair == 1 ? a.rows / 2 : a.rows, cols = pair == 2 ? a.cols / 2 : a.cols;
    return dim3((unsigned)((cols + kTileC - 1) / kTileC), (unsigned)((rows + kTileR - 1) / kTileR),
                (unsigned)a.batch);
  };
  if (a.oa_out != nullptr) {  // (the caller has checked tiles_rowmax_ok: noise none, so spec is 1 or 0)
    if (spec == 1) quant_tile_kernel<TIn, 1, 0, true><<<grid_for(0), 256, 0, st>>>(a);
    else quant_tile_kernel<TIn, 0, 0, true><<<grid_for(0), 256, 0, st>>>(a);
  } else if (spec == 1) {
    quant_tile_kernel<TIn, 1, 0><<<grid_for(0), 256, 0, st>>>(a);
  } else if (spec == 3) {
    quant_tile_kernel<TIn, 3, 0><<<grid_for(0), 256, 0, st>>>(a);
  } else if (spec == 5) {
    // half of a threefry block would be thrown away unless the tile rows/2 further down, whose
    // elements draw from the other half, is quantized by the same workgroup
    const bool natural = a.batch == 1 && a.nsr == a.cols && (a.rows % 2 == 0) && (a.cols % 8 == 0);
    if (natural) quant_tile_kernel<TIn, 5, 1><<<grid_for(1), 256, 0, st>>>(a);
    else quant_tile_kernel<TIn, 5, 0><<<grid_for(0), 256, 0, st>>>(a);
  } else if (spec == 2) {
    // pair the two elements of each threefry block: i and i + total/2 lie rows/2 apart when the
    // noise counters are row-major over [rows, cols], cols/2 apart when over [cols, rows]
    const bool natural = a.batch == 1 && a.nsc == 1 && a.nsr == a.cols && (a.rows % 2 == 0);
    const bool transposed = a.batch == 1 && a.nsr == 1 && a.nsc == a.rows && (a.cols % 16 == 0);
    if (natural) quant_tile_kernel<TIn, 2, 1><<<grid_for(1), 256, 0, st>>>(a);
    else if (transposed) quant_tile_kernel<TIn, 2, 2><<<grid_for(2), 256, 0, st>>>(a);
    else quant_tile_kernel<TIn, 2, 0><<<grid_for(0), 256, 0, st>>>(a);
  } else {
    quant_tile_kernel<TIn, 0, 0><<<grid_for(0), 256, 0, st>>>(a);
  }
  AQTX_HIP_CHECK_LAUNCH("quant_tile_kernel");
  return 0;
}

template <typename TIn>
int dispatch(const QArgs& a, int reduce, int partitionable, int64_t nscales, hipStream_t st) {
  if (reduce == AQTX_REDUCE_COLS) return launch_rows<TIn>(a, partitionable, st);
  return launch_tiles<TIn>(a, reduce, partitionable, nscales, st);
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

// A few very long rows (one scale per image of a convolution's input, say) would leave most of
// the chip idle in the row kernels, which give a row to one wave or workgroup.  Such a plan is the
// same computation as one scale per batch entry of [batch * rows][cols / c][c]: the whole-tensor
// path, which spreads every entry over many workgroups.  Returns true and fills `q` if `p` is
// such a plan.
static bool long_rows_as_batches(const aqtx_quant_plan* p, aqtx_quant_plan* q) {
  if (p->reduce != AQTX_REDUCE_COLS || p->group != 0 || p->transpose_out || p->prescale != AQTX_PRESCALE_NONE ||
      p->out_k_order != AQTX_K_NATURAL)
    return false;
  if (p->batch <= 0 || p->rows <= 0 || p->batch * p->rows > 512 || p->cols < 16384) return false;
  if (p->noise != AQTX_NOISE_NONE && p->batch > 1 && p->noise_stride_batch != p->rows * p->noise_stride_row)
    return false;
  int64_t c = 0;
  for (int64_t cand = 1024; cand >= 64; cand /= 2) {
    if (p->cols % cand == 0) { c = cand; break; }
  }
  if (c == 0) return false;
  *q = *p;
  q->batch = p->batch * p->rows;
  q->rows = p->cols / c;
  q->cols = c;
  q->reduce = AQTX_REDUCE_ALL;
  q->noise_stride_batch = p->noise_stride_row;
  q->noise_stride_row = c * p->noise_stride_col;
  return true;
}

static bool long_rows_as_batches(const aqtx_quant_plan* p, aqtx_quant_plan* q);

extern "C" int64_t aqtx_quantize_other_axis_parts(const aqtx_quant_plan* p) {
  aqtx_quant_plan alt;
  if (p == nullptr || p->scale_given || long_rows_as_batches(p, &alt)) return 0;
  if (rows_colmax_ok(p)) return p->rows < kColmaxBlocks ? p->rows : kColmaxBlocks;
  if (tiles_rowmax_ok(p)) return p->cols / kTileC;
  return 0;
}

extern "C" size_t aqtx_quantize_workspace_bytes(const aqtx_quant_plan* p) {
  aqtx_quant_plan alt;
  if (p != nullptr && long_rows_as_batches(p, &alt)) return aqtx_quantize_workspace_bytes(&alt);
  if (p == nullptr || p->reduce == AQTX_REDUCE_COLS) return 0;
  if (p->batch < 0 || p->rows < 0 || p->cols < 0 || p->group < 0) return 0;
  if (p->reduce < AQTX_REDUCE_ROWS || p->reduce > AQTX_REDUCE_ALL_BATCH) return 0;
  if (p->group > 0 && (p->reduce != AQTX_REDUCE_ROWS || p->rows % p->group != 0)) return 0;
  return (size_t)scale_count(p) * 8;
}

extern "C" int aqtx_quantize(const aqtx_quant_plan* p, const void* x, const float* prescale,
                             void* q, float* scale, void* workspace, size_t workspace_bytes,
                             void* stream) {
  clear_error();
  if (int rc = validate(p)) return rc;
  aqtx_quant_plan alt;
  if (long_rows_as_batches(p, &alt)) return aqtx_quantize(&alt, x, prescale, q, scale, workspace, workspace_bytes, stream);
  const int64_t total = p->batch * p->rows * p->cols;
  if (total == 0) return 0;
  AQTX_REQUIRE(x != nullptr && q != nullptr && scale != nullptr, "aqtx_quantize: NULL buffer");
  AQTX_REQUIRE((p->prescale == AQTX_PRESCALE_NONE) == (prescale == nullptr),
               "aqtx_quantize: prescale pointer does not match plan->prescale");
  AQTX_REQUIRE(p->batch <= 65535, "aqtx_quantize: batch %lld exceeds 65535", (long long)p->batch);
  const size_t need = aqtx_quantize_workspace_bytes(p);
  AQTX_REQUIRE(workspace_bytes >= need && (need == 0 || workspace != nullptr),
               "aqtx_quantize: workspace too small (%zu < %zu)", workspace_bytes, need);
  AQTX_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)q % 16) == 0 &&
                   ((uintptr_t)scale % 4) == 0 &&
                   (prescale == nullptr || ((uintptr_t)prescale % 16) == 0) &&
                   (workspace == nullptr || ((uintptr_t)workspace % 4) == 0),
               "aqtx_quantize: x, q and prescale must be 16-byte aligned");

  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int64_t nscales = scale_count(p);
  QArgs a{};
  a.x = x; a.prescale = prescale; a.q = q; a.scale = scale;
  a.scale_bf16 = (p->scale_typed != nullptr && p->scale_dtype == AQTX_BF16 && !p->scale_given)
                     ? reinterpret_cast<uint16_t*>(p->scale_typed) : nullptr;
  a.batch = p->batch; a.rows = p->rows; a.cols = p->cols;
  a.nsb = p->noise_stride_batch; a.nsr = p->noise_stride_row; a.nsc = p->noise_stride_col;
  a.quant_bound = p->quant_bound; a.clip_bound = p->clip_bound;
  a.noise = p->noise; a.ps_mode = p->prescale; a.psb = p->prescale_stride_batch;
  a.transpose_out = p->transpose_out; a.out_dtype = p->out_dtype;
  a.cbf = p->compute_dtype == AQTX_BF16; a.sbf = p->scale_dtype == AQTX_BF16;
  a.scale_given = p->scale_given;
  a.ws_zeroed = p->workspace_zeroed;
  if (p->other_axis_absmax != nullptr) {
    AQTX_REQUIRE(aqtx_quantize_other_axis_parts(p) > 0,
                 "aqtx_quantize: this plan cannot write other_axis_absmax (aqtx_quantize_other_axis_parts is 0)");
    AQTX_REQUIRE(((uintptr_t)p->other_axis_absmax % 8) == 0, "aqtx_quantize: other_axis_absmax must be 8-byte aligned");
    a.oa_out = reinterpret_cast<uint8_t*>(p->other_axis_absmax);
  }
  if (p->absmax_partials != nullptr) {
    AQTX_REQUIRE(p->in_dtype == AQTX_I8 && p->reduce == AQTX_REDUCE_ROWS && p->group == 0 && p->batch == 1 &&
                     !p->scale_given && p->prescale == AQTX_PRESCALE_NONE && p->absmax_parts > 0 && p->cols % 16 == 0 &&
                     ((uintptr_t)p->absmax_partials % 16) == 0,
                 "aqtx_quantize: absmax_partials (16-byte aligned) go with int8 input, AQTX_REDUCE_ROWS over whole columns (a "
                 "multiple of 16 of them), one batch entry, no prescale and no given scale");
    a.oa_in = reinterpret_cast<const uint8_t*>(p->absmax_partials);
    a.oa_in_parts = p->absmax_parts;
  }
  AQTX_REQUIRE(p->out_k_order == AQTX_K_NATURAL || p->out_k_order == AQTX_K_EVEN_ODD8,
               "aqtx_quantize: unknown out_k_order %d", p->out_k_order);
  if (p->out_k_order == AQTX_K_EVEN_ODD8) {
    AQTX_REQUIRE(p->reduce == AQTX_REDUCE_COLS && !p->transpose_out &&
                     (p->out_dtype == AQTX_I8 || p->out_dtype == AQTX_I4),
                 "aqtx_quantize: out_k_order = EVEN_ODD8 needs AQTX_REDUCE_COLS, an integer out_dtype and no transpose_out");
    a.even_odd8 = 1;
  }
  if (p->noise != AQTX_NOISE_NONE) {
    a.gen = make_bitgen(p->key, p->noise_total, noise_width(p), p->partitionable);
    a.key_dev = p->key_device;
    AQTX_REQUIRE(((uintptr_t)p->key_device % 4) == 0, "aqtx_quantize: key_device is not 4-byte aligned");
  }
  if (p->reduce == AQTX_REDUCE_COLS) {
    a.L = p->group ? p->group : p->cols;
    a.nseg = nscales;
  } else {
    a.ws_absmax = reinterpret_cast<uint32_t*>(workspace);
    // A workspace kept across calls holds the abs-max words (zero between calls) in its first
    // half and the reciprocal scales in its second, whatever the number of scales of a call.
    a.ws_inv = reinterpret_cast<float*>(workspace) +
               (p->workspace_zeroed ? (int64_t)(workspace_bytes / 8) : nscales);
    if (p->reduce == AQTX_REDUCE_ROWS) {
      a.G = p->group ? p->group : p->rows;
      a.ngroups = p->rows / a.G;
      a.ssb = a.ngroups * p->cols; a.ssg = p->cols; a.ssc = 1;
    } else {
      a.G = p->rows; a.ngroups = 1;
      a.ssb = p->reduce == AQTX_REDUCE_ALL ? 1 : 0; a.ssg = 0; a.ssc = 0;
    }
    const int64_t grid_y = p->reduce != AQTX_REDUCE_ROWS
                               ? (p->rows + kTileR - 1) / kTileR
                               : a.ngroups * ((a.G + kAbsRowChunk - 1) / kAbsRowChunk);
    AQTX_REQUIRE(grid_y <= 65535 && (p->rows + kTileR - 1) / kTileR <= 65535,
                 "aqtx_quantize: too many rows for one launch (%lld)", (long long)p->rows);
  }
  switch (p->in_dtype) {
    case AQTX_F32: return dispatch<float>(a, p->reduce, p->partitionable, nscales, st);
    case AQTX_BF16: return dispatch<uint16_t>(a, p->reduce, p->partitionable, nscales, st);
    default: return dispatch<int8_t>(a, p->reduce, p->partitionable, nscales, st);
  }
}

extern "C" int aqtx_dequantize(const aqtx_quant_plan* p, const void* q, const float* scale,
                               void* out, void* stream) {
  clear_error();
  if (int rc = validate(p)) return rc;
  AQTX_REQUIRE(p->in_dtype != AQTX_I8, "aqtx_dequantize: in_dtype names the float result dtype");
  const int64_t total = p->batch * p->rows * p->cols;
  if (total == 0) return 0;
  AQTX_REQUIRE(q != nullptr && scale != nullptr && out != nullptr, "aqtx_dequantize: NULL buffer");
  if (!p->transpose_out && p->group == 0) {
    // q in the order of the result and one scale per row, per column or per (batch) tensor: the
    // 16-columns-per-lane kernel of aqtx_scale_cast, same arithmetic
    aqtx_scale_plan sp{};
    sp.in_dtype = p->out_dtype; sp.out_dtype = p->in_dtype;
    sp.batch = p->batch; sp.rows = p->rows; sp.cols = p->cols;
    sp.factors = 1; sp.factor_dtype[0] = p->scale_dtype;
    if (p->reduce == AQTX_REDUCE_COLS) {
      sp.factor_axis[0] = AQTX_FACTOR_ROWS; sp.factor_stride_b[0] = p->rows;
    } else if (p->reduce == AQTX_REDUCE_ROWS) {
      sp.factor_axis[0] = AQTX_FACTOR_COLS; sp.factor_stride_b[0] = p->cols;
    } else {
      sp.rows = 1; sp.cols = p->rows * p->cols;
      sp.factor_axis[0] = AQTX_FACTOR_ROWS; sp.factor_stride_b[0] = p->reduce == AQTX_REDUCE_ALL ? 1 : 0;
    }
    return aqtx_scale_cast(&sp, q, scale, nullptr, out, stream);
  }
  QArgs a{};
  a.x = q; a.q = out; a.scale = const_cast<float*>(scale);
  a.batch = p->batch; a.rows = p->rows; a.cols = p->cols;
  a.transpose_out = p->transpose_out;
  a.cbf = p->in_dtype == AQTX_BF16; a.sbf = p->scale_dtype == AQTX_BF16;
  // scale index = b*ssb + (r/G)*ssg + (c/L)*ssc
  if (p->reduce == AQTX_REDUCE_COLS) {
    a.L = p->group ? p->group : p->cols; a.G = 1;
    const int64_t per_row = p->cols / a.L;
    a.ssb = p->rows * per_row; a.ssg = per_row; a.ssc = 1;
  } else if (p->reduce == AQTX_REDUCE_ROWS) {
    a.G = p->group ? p->group : p->rows; a.L = 1;
    a.ssb = (p->rows / a.G) * p->cols; a.ssg = p->cols; a.ssc = 1;
  } else {
    a.G = p->rows; a.L = p->cols; a.ssb = p->reduce == AQTX_REDUCE_ALL ? 1 : 0; a.ssg = 0; a.ssc = 0;
  }
  const int fp8_kind = (p->out_dtype == AQTX_E4M3 || p->out_dtype == AQTX_E5M2) ? p->out_dtype : 0;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (p->in_dtype == AQTX_BF16) dequant_kernel<uint16_t><<<dim3(blocks), 256, 0, st>>>(a, fp8_kind);
  else dequant_kernel<float><<<dim3(blocks), 256, 0, st>>>(a, fp8_kind);
  AQTX_HIP_CHECK_LAUNCH("dequant_kernel");
  return 0;
}

extern "C" int aqtx_random_bits(const uint32_t key_host[2], int64_t n, int32_t bit_width,
                                int32_t partitionable, void* out, void* stream) {
  clear_error();
  AQTX_REQUIRE(key_host != nullptr, "aqtx_random_bits: key is NULL");
  AQTX_REQUIRE(bit_width == 16 || bit_width == 32, "aqtx_random_bits: bit_width must be 16 or 32");
  AQTX_REQUIRE(n >= 0 && n < (int64_t)0xFFFFFFFFll, "aqtx_random_bits: n out of range");
  if (n == 0) return 0;
  AQTX_REQUIRE(out != nullptr, "aqtx_random_bits: out is NULL");
  BitGen gen = make_bitgen(key_host, n, bit_width, partitionable);
  random_bits_kernel<<<dim3((unsigned)((n + 255) / 256)), 256, 0,
                       reinterpret_cast<hipStream_t>(stream)>>>(gen, n, out);
  AQTX_HIP_CHECK_LAUNCH("random_bits_kernel");
  return 0;
}

namespace aqtx {
namespace {
__global__ __launch_bounds__(256) void prng_split_kernel(const uint32_t* __restrict__ key, int num, int partitionable,
                                                         uint32_t* __restrict__ out) {
  const int i = (int)(blockIdx.x * 256 + threadIdx.x);  // word i of the 2 * num
  if (i >= 2 * num) return;
  const uint32_t k0 = key[0], k1 = key[1];
  if (partitionable) {
    const U2 b = threefry2x32(k0, k1, 0u, (uint32_t)(i >> 1));
    out[i] = (i & 1) ? b.y : b.x;
  } else {
    BitGen g;
    g.k0 = k0; g.k1 = k1;
    g.nwords = 2u * (uint32_t)num; g.half = (uint32_t)num;
    g.partitionable = 0; g.width = 32;
    out[i] = g.word_original((uint32_t)i);
  }
}
}  // namespace
}  // namespace aqtx

extern "C" int aqtx_prng_split(const uint32_t* key_device, int32_t num, int32_t partitionable, uint32_t* out_device,
                               void* stream) {
  clear_error();
  AQTX_REQUIRE(num >= 0 && num <= (1 << 20), "aqtx_prng_split: num outside 0..2^20");
  if (num == 0) return 0;
  AQTX_REQUIRE(key_device != nullptr && out_device != nullptr, "aqtx_prng_split: NULL argument");
  prng_split_kernel<<<(unsigned)((2 * num + 255) / 256), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
      key_device, num, partitionable, out_device);
  AQTX_HIP_CHECK_LAUNCH("prng_split_kernel");
  return 0;
}

extern "C" int aqtx_prng_split_host(const uint32_t key_host[2], int32_t num, int32_t partitionable,
                                    uint32_t* out_host) {
  clear_error();
  AQTX_REQUIRE(key_host != nullptr && out_host != nullptr, "aqtx_prng_split_host: NULL argument");
  AQTX_REQUIRE(num >= 0, "aqtx_prng_split_host: negative num");
  if (partitionable) {
    for (int32_t i = 0; i < num; ++i) {
      U2 b = threefry2x32(key_host[0], key_host[1], 0u, (uint32_t)i);
      out_host[2 * i] = b.x;
      out_host[2 * i + 1] = b.y;
    }
  } else {
    BitGen g = make_bitgen(key_host, 2 * (int64_t)num, 32, 0);
    for (int32_t i = 0; i < 2 * num; ++i) out_host[i] = g.word_original((uint32_t)i);
  }
  return 0;
}

// aqtx_scale_cast: one elementwise pass from a quantized (or float) tensor to the operand of a float
// contraction, or from the result of one to the dequantized output: cast, then up to two factors that
// have one value per row or per column.  HBM-bound: a lane takes the consecutive columns of one 16-byte
// store; a scalar kernel takes shapes whose rows are not multiples of that many columns or whose buffers
// are not 16-byte aligned.
#include "common.h"

namespace aqtx {
namespace {

struct ScaleArgs {
  const void* x;
  void* out;
  const float* f[2];
  int64_t rows, cols, total;   // rows of one batch entry, columns, elements of the whole tensor
  int64_t fsb[2];              // batch stride of each factor
  int32_t nf;
  int32_t fcols[2];            // 1: one value per column, 0: one value per row
  int32_t fbf[2];              // 1: the factor's values are bf16 values
  int32_t recast[2];
  int32_t recip[2];
  int32_t in_dtype;
  int32_t out_bf;
  float clip;                  // 0: none
  int32_t round;               // 0: none, 1: half to even, 2: floor + 0.5
};

__device__ __forceinline__ float rnd(float x, int bf) { return bf ? round_bf16(x) : x; }

// a factor as it multiplies: itself, or its reciprocal in its own dtype, 1 where that is infinite
__device__ __forceinline__ float factor_value(float f, int recip, int fbf) {
  if (!recip) return f;
  float i = rnd(1.0f / f, fbf);
  if (isinf(i)) i = 1.0f;
  return i;
}

// The products of one element.  RND says at compile time how the running value rounds: 0 = never (float32 out:
// nothing is held in bf16), 1 = after every step (bf16 out and every factor a bf16 value), 2 = as the flags say
// (bf16 out next to a float32 factor: `vbf` follows the dtype jnp's promotion gives the running value).  FINISH:
// the plan clips or rounds at the end.
template <int RND, bool FINISH>
__device__ __forceinline__ float apply(float v, const ScaleArgs& a, float f0, float f1) {
  if constexpr (RND == 2) {
    int vbf = a.out_bf;
    v = rnd(v, vbf);
    if (a.nf > 0) {
      if (a.recast[0]) { v = rnd(v, a.out_bf); vbf = a.out_bf; }
      v = v * factor_value(f0, a.recip[0], a.fbf[0]);
      vbf &= a.fbf[0];
      v = rnd(v, vbf);
    }
    if (a.nf > 1) {
      if (a.recast[1]) { v = rnd(v, a.out_bf); vbf = a.out_bf; }
      v = v * factor_value(f1, a.recip[1], a.fbf[1]);
      vbf &= a.fbf[1];
      v = rnd(v, vbf);
    }
    v = rnd(v, a.out_bf);
  } else {
    v = round_to<RND == 1>(v);
    // (a reciprocal is formed in the factor's own dtype, whatever the product rounds to)
    if (a.nf > 0) v = round_to<RND == 1>(v * factor_value(f0, a.recip[0], RND == 1 ? 1 : a.fbf[0]));
    if (a.nf > 1) v = round_to<RND == 1>(v * factor_value(f1, a.recip[1], RND == 1 ? 1 : a.fbf[1]));
  }
  if constexpr (FINISH) {
    if (a.clip > 0.0f) v = v < -a.clip ? -a.clip : (v > a.clip ? a.clip : v);  // a NaN stays one, as in jnp.clip
    if (a.round == 1) v = rintf(v);
    else if (a.round == 2) v = rnd(floorf(v) + 0.5f, a.out_bf);
  }
  return v;
}

__device__ __forceinline__ float decode_byte(uint32_t byte, int in_dtype) {
  if (in_dtype == AQTX_E4M3) return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
  if (in_dtype == AQTX_E5M2) return __builtin_amdgcn_cvt_f32_bf8((int)byte, 0);
  return (float)(int8_t)byte;
}

// IN: bytes per input element (1, 2 or 4).  One lane = the consecutive columns of one row that make one 16-byte
// store (8 bf16 or 4 float32 results), so that a wave's stores, and its loads, cover whole contiguous lines.
template <int IN, bool OUT_BF, int RND, bool FINISH>
__global__ __launch_bounds__(256) void scale_cast_vec_kernel(const ScaleArgs a) {
  constexpr int E = OUT_BF ? 8 : 4;
  // (several such pieces per lane, for more loads in flight, measured no faster: 14.4 against 14.0 us for 16 M int8
  // values to bf16, where a plain device copy of as many bytes takes as long)
  const int64_t i0 = ((int64_t)blockIdx.x * 256 + threadIdx.x) * E;
  if (i0 >= a.total) return;
  int64_t c0, b, r;  // first column, batch entry, row in it
  if (a.total < (1ll << 31)) {  // 32-bit divisions where they do
    const uint32_t row32 = (uint32_t)i0 / (uint32_t)a.cols;
    c0 = (uint32_t)i0 - row32 * (uint32_t)a.cols;
    const uint32_t b32 = row32 / (uint32_t)a.rows;
    b = b32; r = row32 - b32 * (uint32_t)a.rows;
  } else {
    const int64_t row = i0 / a.cols;
    c0 = i0 - row * a.cols;
    b = row / a.rows; r = row - b * a.rows;
  }

  float v[E];
  if constexpr (IN == 1) {
    uint32_t words[E / 4];
    if constexpr (E == 8) {
      const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(a.x) + i0);
      words[0] = w.x; words[1] = w.y;
    } else {
      words[0] = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const uint8_t*>(a.x) + i0);
    }
#pragma unroll
    for (int j = 0; j < E; ++j) v[j] = decode_byte((words[j >> 2] >> (8 * (j & 3))) & 0xFFu, a.in_dtype);
  } else if constexpr (IN == 2) {
    uint32_t words[E / 2];
    if constexpr (E == 8) {
      const uint4 w = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint16_t*>(a.x) + i0);
      words[0] = w.x; words[1] = w.y; words[2] = w.z; words[3] = w.w;
    } else {
      const uint2 w = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(a.x) + i0);
      words[0] = w.x; words[1] = w.y;
    }
#pragma unroll
    for (int j = 0; j < E; ++j) v[j] = bf16_bits_to_float((uint16_t)(words[j >> 1] >> (16 * (j & 1))));
  } else {
    const float4* p = reinterpret_cast<const float4*>(reinterpret_cast<const float*>(a.x) + i0);
#pragma unroll
    for (int h = 0; h < E / 4; ++h) {
      const float4 w = p[h];
      v[4 * h] = w.x; v[4 * h + 1] = w.y; v[4 * h + 2] = w.z; v[4 * h + 3] = w.w;
    }
  }

  float f[2][E];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    if (i < a.nf) {
      if (a.fcols[i]) {
        const float4* p = reinterpret_cast<const float4*>(a.f[i] + b * a.fsb[i] + c0);
#pragma unroll
        for (int h = 0; h < E / 4; ++h) {
          const float4 w = p[h];
          f[i][4 * h] = w.x; f[i][4 * h + 1] = w.y; f[i][4 * h + 2] = w.z; f[i][4 * h + 3] = w.w;
        }
      } else {
        const float s = a.f[i][b * a.fsb[i] + r];
#pragma unroll
        for (int j = 0; j < E; ++j) f[i][j] = s;
      }
    } else {
#pragma unroll
      for (int j = 0; j < E; ++j) f[i][j] = 1.0f;
    }
  }
#pragma unroll
  for (int j = 0; j < E; ++j) v[j] = apply<RND, FINISH>(v[j], a, f[0][j], f[1][j]);

  if constexpr (OUT_BF) {
    uint32_t w[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) w[j] = (uint32_t)bf16_bits(v[2 * j]) | ((uint32_t)bf16_bits(v[2 * j + 1]) << 16);
    *reinterpret_cast<uint4*>(reinterpret_cast<uint16_t*>(a.out) + i0) = make_uint4(w[0], w[1], w[2], w[3]);
  } else {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(a.out) + i0) = make_float4(v[0], v[1], v[2], v[3]);
  }
}

// one element per lane: any shape, any alignment
__global__ __launch_bounds__(256) void scale_cast_scalar_kernel(const ScaleArgs a) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= a.total) return;
  const int64_t row = i / a.cols, c = i - row * a.cols;
  const int64_t b = row / a.rows, r = row - b * a.rows;
  float v;
  if (a.in_dtype == AQTX_F32) v = reinterpret_cast<const float*>(a.x)[i];
  else if (a.in_dtype == AQTX_BF16) v = bf16_bits_to_float(reinterpret_cast<const uint16_t*>(a.x)[i]);
  else v = decode_byte(reinterpret_cast<const uint8_t*>(a.x)[i], a.in_dtype);
  float f[2] = {1.0f, 1.0f};
  for (int k = 0; k < a.nf; ++k) f[k] = a.f[k][b * a.fsb[k] + (a.fcols[k] ? c : r)];
  v = apply<2, true>(v, a, f[0], f[1]);
  if (a.out_bf) reinterpret_cast<uint16_t*>(a.out)[i] = bf16_bits(v);
  else reinterpret_cast<float*>(a.out)[i] = v;
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_scale_cast(const aqtx_scale_plan* p, const void* x, const float* f0, const float* f1,
                               void* out, void* stream) {
  clear_error();
  AQTX_REQUIRE(p != nullptr, "aqtx_scale_cast: plan is NULL");
  const bool in_byte = p->in_dtype == AQTX_I8 || p->in_dtype == AQTX_I4 || p->in_dtype == AQTX_E4M3 ||
                       p->in_dtype == AQTX_E5M2;
  AQTX_REQUIRE(in_byte || is_float_dtype(p->in_dtype), "aqtx_scale_cast: unsupported in_dtype %d", p->in_dtype);
  AQTX_REQUIRE(is_float_dtype(p->out_dtype), "aqtx_scale_cast: out_dtype must be f32 or bf16, got %d", p->out_dtype);
  AQTX_REQUIRE(p->batch >= 0 && p->rows >= 0 && p->cols >= 0, "aqtx_scale_cast: negative shape");
  AQTX_REQUIRE(p->factors >= 0 && p->factors <= 2, "aqtx_scale_cast: factors must be 0, 1 or 2, got %d", p->factors);
  const float* fs[2] = {f0, f1};
  ScaleArgs a{};
  for (int i = 0; i < p->factors; ++i) {
    AQTX_REQUIRE(p->factor_axis[i] == AQTX_FACTOR_ROWS || p->factor_axis[i] == AQTX_FACTOR_COLS,
                 "aqtx_scale_cast: unknown factor_axis %d", p->factor_axis[i]);
    AQTX_REQUIRE(is_float_dtype(p->factor_dtype[i]), "aqtx_scale_cast: factor_dtype must be f32 or bf16, got %d",
                 p->factor_dtype[i]);
    AQTX_REQUIRE(p->factor_stride_b[i] >= 0, "aqtx_scale_cast: negative factor stride");
    a.f[i] = fs[i];
    a.fsb[i] = p->factor_stride_b[i];
    a.fcols[i] = p->factor_axis[i] == AQTX_FACTOR_COLS;
    a.fbf[i] = p->factor_dtype[i] == AQTX_BF16;
    a.recast[i] = p->factor_recast[i] != 0;
    a.recip[i] = p->factor_reciprocal[i] != 0;
  }
  AQTX_REQUIRE(p->finish_clip >= 0.0f, "aqtx_scale_cast: negative finish_clip");
  AQTX_REQUIRE(p->finish_round >= 0 && p->finish_round <= 2, "aqtx_scale_cast: finish_round must be 0, 1 or 2, got %d",
               p->finish_round);
  a.clip = p->finish_clip; a.round = p->finish_round;
  const int64_t total = p->batch * p->rows * p->cols;
  if (total == 0) return 0;
  AQTX_REQUIRE(x != nullptr && out != nullptr, "aqtx_scale_cast: NULL buffer");
  for (int i = 0; i < p->factors; ++i)
    AQTX_REQUIRE(fs[i] != nullptr && ((uintptr_t)fs[i] % 4) == 0, "aqtx_scale_cast: factor %d is NULL or unaligned", i);
  const size_t isz = dtype_size(p->in_dtype), osz = dtype_size(p->out_dtype);
  AQTX_REQUIRE(((uintptr_t)x % isz) == 0 && ((uintptr_t)out % osz) == 0, "aqtx_scale_cast: buffer not element aligned");
  a.x = x; a.out = out;
  a.rows = p->rows; a.cols = p->cols; a.total = total;
  a.nf = p->factors; a.in_dtype = p->in_dtype; a.out_bf = p->out_dtype == AQTX_BF16;

  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const int per_lane = a.out_bf ? 8 : 4;  // results of one 16-byte store
  bool vec = p->cols % per_lane == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  for (int i = 0; i < p->factors; ++i)
    if (a.fcols[i]) vec = vec && ((uintptr_t)fs[i] % 16) == 0 && a.fsb[i] % 4 == 0;
  if (vec) {
    const int64_t blocks = (total / per_lane + 255) / 256;
    AQTX_REQUIRE(blocks < (1ll << 31), "aqtx_scale_cast: tensor too large for one launch");
    const dim3 grid((unsigned)blocks);
    // how the running value rounds, known per launch: never (float32 out), after every step (bf16 all through),
    // or by the flags (a float32 factor next to a bf16 result)
    bool all_bf = a.out_bf;
    for (int i = 0; i < p->factors; ++i) all_bf = all_bf && a.fbf[i];
    const int rnd_mode = !a.out_bf ? 0 : all_bf ? 1 : 2;
    const bool finish = a.clip > 0.0f || a.round != 0;
#define AQTX_SC3(IN, OUT, RND) do { if (finish) scale_cast_vec_kernel<IN, OUT, RND, true><<<grid, 256, 0, st>>>(a); \
                                    else scale_cast_vec_kernel<IN, OUT, RND, false><<<grid, 256, 0, st>>>(a); } while (0)
#define AQTX_SC(IN) do { if (rnd_mode == 0) AQTX_SC3(IN, false, 0); else if (rnd_mode == 1) AQTX_SC3(IN, true, 1); \
                         else AQTX_SC3(IN, true, 2); } while (0)
    if (isz == 1) AQTX_SC(1); else if (isz == 2) AQTX_SC(2); else AQTX_SC(4);
#undef AQTX_SC
#undef AQTX_SC3
    AQTX_HIP_CHECK_LAUNCH("scale_cast_vec_kernel");
  } else {
    const int64_t blocks = (total + 255) / 256;
    AQTX_REQUIRE(blocks < (1ll << 31), "aqtx_scale_cast: tensor too large for one launch");
    scale_cast_scalar_kernel<<<dim3((unsigned)blocks), 256, 0, st>>>(a);
    AQTX_HIP_CHECK_LAUNCH("scale_cast_scalar_kernel");
  }
  return 0;
}

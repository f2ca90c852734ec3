// Weight-only serving: a float (bf16) activation [m <= 64][k] against a frozen int8 or packed int4 weight
// [n][k] with one scale per output channel,
//   out[m][n] = dequant( sum_k x[m][k] * float(w[n][k]) ),
// the contraction the reference runs when only the rhs is quantized (aqt/jax/v2/aqt_dot_general.py:843-958
// with a float lhs: the int8 qvalue is promoted to the float dtype, lax.dot_general contracts in it, the
// rhs scale multiplies the output).  Bytes per call = the weight, streamed once from HBM; the weight bytes
// are converted to bf16 (exactly) in registers on their way into v_mfma_f32_16x16x32_bf16, the
// activations are the MFMA's other operand as they lie in memory.  Sums are float32 (K split over the four
// waves of a workgroup, added in wave order), so results agree with the library product on the promoted
// weight to float32 summation order, not bit for bit.
//
// A workgroup owns 16 NB weight rows and all 16 MB tokens; wave w walks the w-th quarter of K in steps of
// one weight fragment (16 rows x 64 bytes: 64 k of int8, 128 k of packed int4), D steps in flight.  Lane
// (r, c) = (lane % 16, lane / 16) holds 16 bytes of weight row r: k 16c..16c+15 (int8) or 32c..32c+31
// (packed) of the step, i.e. two (four) MFMA operands of 8 bf16 after conversion, and reads the same k of
// token r: 32 (64) contiguous bytes.  The weight is the MFMA's first operand, so a lane ends with four
// consecutive outputs n of one token.
//
// Every workgroup reads all of its tokens' activations (from L2), so with many tokens and a narrow weight
// (few 64-row tiles) the activation traffic of 16-row tiles is a multiple of the weight's.  Given a workspace,
// such calls keep the 64-row tiles and cut K into slices instead (grid.y): a workgroup leaves its float32
// partial sums in slab s of the workspace, and decode_wo_sum_kernel adds the slabs in slice order and applies
// the epilogue: still one fixed summation order.
#include <type_traits>

#include "common.h"

namespace aqtx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v2bf __attribute__((ext_vector_type(2)));
typedef float v2f __attribute__((ext_vector_type(2)));

constexpr uint32_t kRsrcWord3 = 0x00020000u;  // raw buffer, 32-bit data format (gfx9)
constexpr int kOob = 0x7FFFFFF0;              // offset that is out of range for every buffer

struct WoArgs {
  const uint8_t* x;      // bf16 [m][k]
  const uint8_t* w;      // int8 [n][k], packed int4 [n][k/2], or either in fragment order
  const float* w_scale;  // [n]
  void* out;             // [m][n]
  int m, n, k;
  int out_bf16, ws_bf16;
  int w_frag, w_steps;
  int splits, k_slice;   // slices of K (grid.y) and their length, a multiple of four weight fragment steps
  float* slabs;          // [splits][m][n] partial sums when splits > 1
};

__device__ __forceinline__ float rnd(float v, int bf) { return bf ? round_bf16(v) : v; }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, kRsrcWord3);
}

// Two floats -> one word of two bf16 (low half = a); exact for the small integers converted here.
__device__ __forceinline__ uint32_t pack_bf16(float a, float b) {
  const v2bf h = __builtin_convertvector(v2f{a, b}, v2bf);
  return __builtin_bit_cast(uint32_t, h);
}

// 16 weight bytes -> NOPS MFMA operands of 8 bf16 in k order.
template <bool PACKED>
__device__ __forceinline__ void weight_operands(const v4i w, v8bf (&op)[PACKED ? 4 : 2]) {
  if constexpr (!PACKED) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      uint32_t u[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int word = w[2 * j + (q >> 1)];
        const int sh = 16 * (q & 1);
        u[q] = pack_bf16((float)(int8_t)(word >> sh), (float)(int8_t)(word >> (sh + 8)));
      }
      op[j] = __builtin_bit_cast(v8bf, v4i{(int)u[0], (int)u[1], (int)u[2], (int)u[3]});
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {  // word j: nibbles 0..7 = k 8j .. 8j+7, low nibble of a byte = even k
      const int word = w[j];
      uint32_t u[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const float lo = (float)((word << (28 - 8 * q)) >> 28);        // nibble 2q, sign extended
        const float hi = (float)((word << (24 - 8 * q)) >> 28);        // nibble 2q + 1
        u[q] = pack_bf16(lo, hi);
      }
      op[j] = __builtin_bit_cast(v8bf, v4i{(int)u[0], (int)u[1], (int)u[2], (int)u[3]});
    }
  }
}

// The contraction's result in the activation dtype, times the rhs scale in the promoted dtype, final cast;
// four consecutive outputs n of token mm.
__device__ __forceinline__ void wo_store(const WoArgs& d, int mm, int nn, const v4f total, bool wide_ok) {
  float f[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float ws = d.w_scale[(nn + e) < d.n ? (nn + e) : (d.n - 1)];
    float v = round_bf16(total[e]);
    v = rnd(v * ws, d.ws_bf16);
    f[e] = rnd(v, d.out_bf16);
  }
  const int64_t o = (int64_t)mm * d.n + nn;
  if (wide_ok) {
    if (d.out_bf16) {
      uint2 v;
      v.x = (uint32_t)bf16_bits(f[0]) | ((uint32_t)bf16_bits(f[1]) << 16);
      v.y = (uint32_t)bf16_bits(f[2]) | ((uint32_t)bf16_bits(f[3]) << 16);
      *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(d.out) + o) = v;
    } else {
      *reinterpret_cast<float4*>(reinterpret_cast<float*>(d.out) + o) = make_float4(f[0], f[1], f[2], f[3]);
    }
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (nn + e < d.n) {
        if (d.out_bf16) reinterpret_cast<uint16_t*>(d.out)[o + e] = bf16_bits(f[e]);
        else reinterpret_cast<float*>(d.out)[o + e] = f[e];
      }
  }
}

template <int MB, int NB, int D, bool PACKED>
__global__ __launch_bounds__(256) void decode_wo_kernel(const WoArgs d) {
  constexpr int T = MB * NB;             // output tiles of 16 x 16 per workgroup
  constexpr int TPW = (T + 3) / 4;       // tiles a wave dequantizes at the end
  constexpr int KS = PACKED ? 128 : 64;  // k of one weight fragment step
  constexpr int KL = KS / 4;             // k of one lane's 16 bytes
  constexpr int NOPS = KL / 8;           // MFMA operands per lane and step
  __shared__ v4f red[4][T][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int n0 = (int)blockIdx.x * 16 * NB;
  const int kb = PACKED ? d.k / 2 : d.k;  // bytes of one weight row
  const int s_lo = (int)blockIdx.y * d.k_slice;
  const int s_hi = (s_lo + d.k_slice) < d.k ? (s_lo + d.k_slice) : d.k;
  const int kq = d.k_slice / 4;
  const int k_lo = s_lo + wave * kq;
  const int k_hi = (k_lo + kq) < s_hi ? (k_lo + kq) : s_hi;

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, d.w_frag ? (int64_t)((d.n + 15) / 16) * d.w_steps * 1024 : (int64_t)d.n * kb);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.x, (int64_t)d.m * d.k * 2);
  int wbase[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int row = n0 + nb * 16 + r;
    wbase[nb] = d.w_frag ? (int)(blockIdx.x * NB + nb) * d.w_steps * 1024 + lane * 16  // past n: reads zeros
                         : (row < d.n ? row : d.n - 1) * kb + c * 16;  // clamped; such columns are never stored
  }
  unsigned xbase[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int t = mb * 16 + r;
    xbase[mb] = t < d.m ? (unsigned)(t * d.k + c * KL) * 2u : (unsigned)kOob;  // tokens past m read zeros
  }

  v4f acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = v4f{0.0f, 0.0f, 0.0f, 0.0f};

  const unsigned wstep = d.w_frag ? 1024u : 64u;
  v4i wf[D][NB], xf[D][MB][NOPS];
  // Steps past the end of the wave's range and lanes past the end of K read zeros: their offsets get the
  // out-of-range bits ORed in (no memory access, no branch)
  auto issue = [&](auto stream_c, const int slot, int ko) {
    // (where the weight stream is what bounds the kernel: not for packed int4, bound by the conversion, nor for
    // more than 16 tokens; both measured 5-10 % slower with the hint)
    constexpr int kPolicy = (decltype(stream_c)::value && !PACKED && MB == 1) ? kStreamOnce : 0;
    const unsigned dead = (ko + c * KL < k_hi) ? 0u : (unsigned)kOob;  // a lane's KL values are all inside or all outside
    const unsigned wk = (unsigned)(ko / KS) * wstep;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[slot][nb] = __builtin_amdgcn_raw_buffer_load_b128(rw, (int)(((unsigned)wbase[nb] + wk) | dead), 0, kPolicy);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int j = 0; j < NOPS; ++j)
        xf[slot][mb][j] = __builtin_amdgcn_raw_buffer_load_b128(
            rx, (int)((xbase[mb] + (unsigned)ko * 2u + (unsigned)j * 16u) | dead), 0, 0);
  };
  auto multiply = [&](const int slot) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      v8bf wop[NOPS];
      weight_operands<PACKED>(wf[slot][nb], wop);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int j = 0; j < NOPS; ++j)
          acc[mb][nb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wop[j], __builtin_bit_cast(v8bf, xf[slot][mb][j]),
                                                                acc[mb][nb], 0, 0, 0);
    }
  };
  const int nsteps = kq / KS;
  auto step_k = [&](int i) { return i < nsteps ? k_lo + i * KS : 0x3FFFFF00; };
  // streaming hint on the weight loads when a wave load is a whole KiB fragment, chosen once outside the loop
  auto walk = [&](auto stream_c) {
#pragma unroll
    for (int s = 0; s < D; ++s) issue(stream_c, s, step_k(s));
    __builtin_amdgcn_sched_barrier(0);
    for (int i = 0; i < nsteps; i += D) {
#pragma unroll
      for (int s = 0; s < D; ++s) {
        multiply(s);
        __builtin_amdgcn_sched_barrier(0);
        issue(stream_c, s, step_k(i + D + s));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  if (d.w_frag) walk(std::true_type{}); else walk(std::false_type{});
  // lane holds C[n = n0 + nb*16 + 4c + e][m = mb*16 + r] in acc[mb][nb][e]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) red[wave][mb * NB + nb][lane] = acc[mb][nb];
  __syncthreads();
  const bool wide_ok = (d.n % 4) == 0;  // 4 consecutive outputs of a row are then 8 / 16-byte aligned
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int t = wave + 4 * j;
    if (T % 4 != 0 && t >= T) break;  // fewer tiles than waves (uniform per wave)
    const v4f total = ((red[0][t][lane] + red[1][t][lane]) + red[2][t][lane]) + red[3][t][lane];
    const int mm = (t / NB) * 16 + r, nn = n0 + (t % NB) * 16 + 4 * c;
    if (mm >= d.m || nn >= d.n) continue;
    if (d.splits > 1) {
      float* dst = d.slabs + ((int64_t)blockIdx.y * d.m + mm) * d.n + nn;
      if (wide_ok) *reinterpret_cast<float4*>(dst) = make_float4(total[0], total[1], total[2], total[3]);
      else for (int e = 0; e < 4 && nn + e < d.n; ++e) dst[e] = total[e];
      continue;
    }
    wo_store(d, mm, nn, total, wide_ok);
  }
}

// out = epilogue(slab 0 + slab 1 + ...), the slabs added in slice order; thread -> four consecutive n of one token
__global__ __launch_bounds__(256) void decode_wo_sum_kernel(const WoArgs d) {
  const int64_t quads = (d.n + 3) / 4;
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (id >= quads * d.m) return;
  const int mm = (int)(id / quads), nn = (int)(id % quads) * 4;
  const bool wide_ok = (d.n % 4) == 0;
  v4f total = v4f{0.0f, 0.0f, 0.0f, 0.0f};
  for (int sl = 0; sl < d.splits; ++sl) {
    const float* src = d.slabs + ((int64_t)sl * d.m + mm) * d.n + nn;
    v4f part = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    if (wide_ok) {
      const float4 t = *reinterpret_cast<const float4*>(src);
      part = v4f{t.x, t.y, t.z, t.w};
    } else {
      for (int e = 0; e < 4 && nn + e < d.n; ++e) part[e] = src[e];
    }
    total = sl == 0 ? part : total + part;
  }
  wo_store(d, mm, nn, total, wide_ok);
}

template <int MB, int NB, int D>
void launch_wo(const WoArgs& d, bool packed, dim3 grid, hipStream_t st) {
  if (packed) decode_wo_kernel<MB, NB, D, true><<<grid, 256, 0, st>>>(d);
  else decode_wo_kernel<MB, NB, D, false><<<grid, 256, 0, st>>>(d);
}

// Launch shape for a plan: token blocks, weight blocks per workgroup, slices of K and their length.
struct WoShape { int mb, nb, splits, k_slice; };

WoShape wo_shape(const aqtx_decode_plan* p, bool with_workspace) {
  const bool pk = p->w_dtype == AQTX_I4P;
  const int ks = pk ? 128 : 64;
  WoShape s;
  s.mb = p->m <= 16 ? 1 : p->m <= 32 ? 2 : 4;
  // the tallest weight tile of 64 / 32 / 16 rows that still gives most CUs a workgroup
  s.nb = 4;
  while (s.nb > 1 && (p->n + 16 * s.nb - 1) / (16 * s.nb) < 192) s.nb /= 2;
  s.splits = 1;
  const int64_t tiles64 = (p->n + 63) / 64;
  if (with_workspace && s.nb < 4 && (p->m > 32 || (p->m > 16 && s.nb == 1 && p->k >= 8192))) {
    // many tokens against a narrow weight: 64-row tiles (a quarter of the activation reads of 16-row tiles)
    // and slices of K until about 256 workgroups exist, each slice at least 1024 of k.  Measured: it pays
    // from 33 tokens on, and from 17 where 16-row tiles would walk a long k (the second launch costs 2 us)
    int64_t want = (256 + tiles64 - 1) / tiles64;
    want = want > 8 ? 8 : want;
    want = want > p->k / 1024 ? p->k / 1024 : want;
    if (want >= 2) { s.nb = 4; s.splits = (int)want; }
  }
  if (const int t = p->tuning & 7; t == 1 || t == 2 || t == 4) s.nb = t;
  if (const int t = (p->tuning >> 4) & 15; with_workspace && t >= 1 && t <= 8 && t <= p->k / (4 * ks)) s.splits = t;
  const int64_t per = (p->k + s.splits - 1) / s.splits;
  s.k_slice = (int)((per + 4 * ks - 1) / (4 * ks) * (4 * ks));
  s.splits = (int)((p->k + s.k_slice - 1) / s.k_slice);
  return s;
}

int validate_wo(const aqtx_decode_plan* p) {
  AQTX_REQUIRE(p != nullptr, "aqtx_decode_weight_only: plan is NULL");
  AQTX_REQUIRE(p->m >= 0 && p->n >= 0 && p->k >= 0, "aqtx_decode_weight_only: negative shape");
  AQTX_REQUIRE(p->m <= 64, "aqtx_decode_weight_only: m = %lld exceeds 64", (long long)p->m);
  AQTX_REQUIRE(p->w_dtype == AQTX_I8 || p->w_dtype == AQTX_I4 || p->w_dtype == AQTX_I4P,
               "aqtx_decode_weight_only: w_dtype must be int8, int4 in int8 containers or packed int4");
  const bool pk = p->w_dtype == AQTX_I4P;
  const int64_t kmul = pk ? 32 : 16;
  AQTX_REQUIRE(p->k > 0 && p->k % kmul == 0, "aqtx_decode_weight_only: k = %lld must be a positive multiple of %lld",
               (long long)p->k, (long long)kmul);
  AQTX_REQUIRE(p->x_dtype == AQTX_BF16, "aqtx_decode_weight_only: activations must be bf16");
  AQTX_REQUIRE(is_float_dtype(p->w_scale_dtype) && is_float_dtype(p->out_dtype),
               "aqtx_decode_weight_only: dtypes must be bf16 or f32");
  AQTX_REQUIRE(p->n * p->k < (1ll << 31) - 64 && p->m * p->n < (1ll << 31) && p->m * p->k * 2 < (1ll << 31),
               "aqtx_decode_weight_only: tensors larger than 2 GiB are not addressable with 32-bit offsets");
  AQTX_REQUIRE(p->w_layout == AQTX_W_ROWS || p->w_layout == AQTX_W_FRAGMENTS,
               "aqtx_decode_weight_only: unknown w_layout %d", p->w_layout);
  AQTX_REQUIRE(p->w_layout == AQTX_W_ROWS || (p->n + 15) / 16 * ((p->k + 63) / 64) * 1024 < (1ll << 31) - 64,
               "aqtx_decode_weight_only: fragment-ordered weight larger than 2 GiB");
  return 0;
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" size_t aqtx_decode_weight_only_workspace_bytes(const aqtx_decode_plan* p) {
  clear_error();
  if (validate_wo(p) != 0 || p->m == 0 || p->n == 0) return 0;
  const WoShape s = wo_shape(p, true);
  return s.splits > 1 ? (size_t)s.splits * (size_t)p->m * (size_t)p->n * 4 : 0;
}

extern "C" int aqtx_decode_weight_only(const aqtx_decode_plan* p, const void* x, const void* w, const float* w_scale,
                                       void* out, void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  if (int rc = validate_wo(p)) return rc;
  const bool pk = p->w_dtype == AQTX_I4P;
  if (p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(x != nullptr && w != nullptr && w_scale != nullptr && out != nullptr, "aqtx_decode_weight_only: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)w % 16) == 0 && ((uintptr_t)x % 16) == 0, "aqtx_decode_weight_only: x and w must be 16-byte aligned");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)out % (4 * esz)) == 0 || p->n % 4 != 0, "aqtx_decode_weight_only: out must be aligned to four elements");
  // slices of K only with a workspace that holds their partial sums (the call works without one)
  WoShape s = wo_shape(p, workspace != nullptr);
  if (s.splits > 1 && (workspace_bytes < (size_t)s.splits * p->m * p->n * 4 || ((uintptr_t)workspace % 16) != 0))
    s = wo_shape(p, false);

  WoArgs d{};
  d.x = reinterpret_cast<const uint8_t*>(x);
  d.w = reinterpret_cast<const uint8_t*>(w);
  d.w_scale = w_scale; d.out = out;
  d.m = (int)p->m; d.n = (int)p->n; d.k = (int)p->k;
  d.out_bf16 = p->out_dtype == AQTX_BF16;
  d.ws_bf16 = p->w_scale_dtype == AQTX_BF16;
  d.w_frag = p->w_layout == AQTX_W_FRAGMENTS;
  d.w_steps = (int)(((pk ? p->k / 2 : p->k) + 63) / 64);
  d.splits = s.splits; d.k_slice = s.k_slice;
  d.slabs = reinterpret_cast<float*>(workspace);
  const int nb = s.nb;
  const dim3 grid((unsigned)((p->n + 16 * nb - 1) / (16 * nb)), (unsigned)s.splits);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
#define AQTX_WO(M)                                                \
  do {                                                            \
    if (nb == 4) launch_wo<M, 4, (M == 4 ? 2 : 4)>(d, pk, grid, st); \
    else if (nb == 2) launch_wo<M, 2, 4>(d, pk, grid, st);        \
    else launch_wo<M, 1, 4>(d, pk, grid, st);                     \
  } while (0)
  if (s.mb == 1) AQTX_WO(1); else if (s.mb == 2) AQTX_WO(2); else AQTX_WO(4);
#undef AQTX_WO
  AQTX_HIP_CHECK_LAUNCH("decode_wo_kernel");
  if (s.splits > 1) {
    const int64_t quads = (int64_t)((p->n + 3) / 4) * p->m;
    decode_wo_sum_kernel<<<dim3((unsigned)((quads + 255) / 256)), 256, 0, st>>>(d);
    AQTX_HIP_CHECK_LAUNCH("decode_wo_sum_kernel");
  }
  return 0;
}

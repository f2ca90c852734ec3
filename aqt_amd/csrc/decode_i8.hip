// Serving-shape contraction: out[m, n] = dequant( quant(x)[m, :] . W[n, :] ) for m <= 64 rows of
// activations against a pre-quantized int8 weight stored [n, k] (contraction axis contiguous).
//
// The weight is read exactly once and dominates the traffic, so the kernels are built around
// streaming W from HBM with every lane fetching 16 contiguous bytes straight into the operand
// registers of v_mfma_i32_16x16x64_i8 (lane -> row lane&15, bytes 16*(lane>>4).. of a 64-byte
// k step: 16 rows x 64 B per wave instruction, whole 64-byte sectors).  The activations are
// quantized first by the row kernel of aqtx_quantize (same arithmetic as training), then:
//   K split : one workgroup per 16 weight rows, its 4 waves split K and meet in LDS; the
//             quantized activations come from L2 (m <= 16, or a weight with few rows);
//   whole K : one workgroup per 64 weight rows; two groups of 4 waves (16 rows per wave) take half
//             of K each and meet in LDS; the activations are staged chunk by chunk in LDS and
//             shared by the waves of a group, the weights are requested three chunks ahead
//             (16 < m <= 64 and n >= 12288).  K is never split across workgroups: a partial-sum
//             exchange inside one launch would need device-scope release/acquire, which
//             flushes and invalidates the per-XCD L2s.
#include "common.h"

namespace aqtx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr uint32_t kBufferRsrcWord3 = 0x00020000u;  // raw buffer, 32-bit data format (gfx9)
constexpr int kOob = 0x7FFFFFF0;                     // offset that is out of range for every buffer

struct DecodeArgs {
  const int8_t* xq;       // [m][k]
  const int8_t* w;        // [n][k]
  const float* x_scale;   // [m]
  const float* w_scale;   // [n]
  void* out;              // [m][n]
  int m, n, k;
  int out_bf16, xs_bf16, ws_bf16;
  int acc_shift;  // 4 when the weight operand holds 16 * w (unpacked nibbles), else 0
  // the fused kernel quantizes the activations itself
  const void* x;          // [m][k] bf16 or f32
  int8_t* xq_out;         // optional [m][k]
  float* x_scale_out;     // [m]
  float quant_bound, clip_bound;
  int x_bf16;
};

__device__ __forceinline__ float rnd(float x, int bf) { return bf ? round_bf16(x) : x; }

// QTensor.dequant: cast the accumulator, multiply by the lhs scale, then the rhs scale, each
// product in the promoted dtype of its operands, final cast.
__device__ __forceinline__ void store_out_scaled(const DecodeArgs& d, int mm, int nn, int acc, float xs) {
  float f = rnd((float)(acc >> d.acc_shift), d.out_bf16);  // exact: acc is a multiple of 16 then
  const int p1 = d.out_bf16 & d.xs_bf16;
  f = rnd(f * xs, p1);
  f = rnd(f * d.w_scale[nn], p1 & d.ws_bf16);
  f = rnd(f, d.out_bf16);
  const int64_t o = (int64_t)mm * d.n + nn;
  if (d.out_bf16) reinterpret_cast<uint16_t*>(d.out)[o] = bf16_bits(f);
  else reinterpret_cast<float*>(d.out)[o] = f;
}
__device__ __forceinline__ void store_out(const DecodeArgs& d, int mm, int nn, int acc) {
  store_out_scaled(d, mm, nn, acc, d.x_scale[mm]);
}

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, kBufferRsrcWord3);
}

// ---- K split inside the workgroup ---------------------------------------------------------------
// One workgroup per 16 weight rows; its 4 waves take a quarter of K each and meet in LDS.  The
// quantized activations are read straight from L2 as MFMA operands (MB blocks of 16 rows), so
// the L2 traffic is (1 + MB) times the weight bytes: the shape for m <= 16, and for larger m
// when the weight has too few rows to fill the chip with whole-K waves.
template <int MB, int U>  // U: 64-byte k steps in flight per wave
__global__ __launch_bounds__(256) void decode_ksplit_kernel(const DecodeArgs d) {
  __shared__ int red[4][MB * 16][16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = (n0 + r) < d.n ? (n0 + r) : (d.n - 1);  // clamped; such columns are never stored

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, (int64_t)d.n * d.k);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.xq, (int64_t)d.m * d.k);
  const int kq = ((d.k + 3) / 4 + 63) / 64 * 64;  // K range of one wave, whole 64-byte steps
  const int k_lo = wave * kq;
  const int k_hi = (k_lo + kq) < d.k ? (k_lo + kq) : d.k;
  const int wbase = nrow * d.k + c * 16;
  int xbase[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) xbase[mb] = (mb * 16 + r) < d.m ? (mb * 16 + r) * d.k + c * 16 : kOob;

  v4i acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = v4i{0, 0, 0, 0};
  for (int kk = k_lo; kk < k_hi; kk += 64 * U) {
    v4i wf[U], xf[U][MB];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ko = kk + u * 64;
      const bool ok = ko + c * 16 < k_hi;
      wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, ok ? wbase + ko : kOob, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        xf[u][mb] = __builtin_amdgcn_raw_buffer_load_b128(rx, (ok && xbase[mb] != kOob) ? xbase[mb] + ko : kOob, 0, 0);
    }
    // Keep every load of the batch in flight before the first MFMA waits for one: left alone,
    // the scheduler interleaves them to save registers and the wave stalls on memory latency.
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][mb], wf[u], acc[mb], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
  // lane holds C[m = mb*16 + 4c + e][n = r]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][mb * 16 + 4 * c + e][r] = acc[mb][e];
  __syncthreads();
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int mm = mb * 16 + (tid >> 4), nn = n0 + (tid & 15);
    if (mm < d.m && nn < d.n) {
      const int s = red[0][mm][tid & 15] + red[1][mm][tid & 15] + red[2][mm][tid & 15] + red[3][mm][tid & 15];
      store_out(d, mm, nn, s);
    }
  }
}

// A word of eight packed int4 (low nibble = even k) -> two words of int8 holding 16 * value.
__device__ __forceinline__ void unpack_i4x8(uint32_t w, int& lo, int& hi) {
  const uint32_t ev = (w << 4) & 0xF0F0F0F0u;  // k0 k2 k4 k6
  const uint32_t od = w & 0xF0F0F0F0u;         // k1 k3 k5 k7
  lo = (int)__builtin_amdgcn_perm(od, ev, 0x05010400u);  // k0 k1 k2 k3
  hi = (int)__builtin_amdgcn_perm(od, ev, 0x07030602u);  // k4 k5 k6 k7
}

// ---- few rows: activation quantisation inside the contraction kernel ------------------------------
// For a handful of tokens the separate quantize launch costs as much as a third of the call.
// Here every workgroup quantizes the activations itself (they come from L2: ROWS * k values),
// keeps the int8 rows in LDS and multiplies them with its 16 weight rows as the K-split kernel
// does.  The first batch of weight loads is issued before the quantisation so that HBM latency
// overlaps it.  Same arithmetic as the row kernel of aqtx_quantize: abs-max over the row,
// scale = dtype(absmax / bound), inv = dtype(1 / scale), q = rint(clip(dtype(x * inv))).
// Workgroup 0 also writes the scales and, when asked, the quantized activations.
// LDS rows are k rounded up to 256 bytes long; the 16-byte piece j of row i sits at piece
// j ^ (i & 15) of its 16-piece group, so the 16 lanes of a fragment read hit all 64 banks.
// PACKED: int4 weights two per byte; a lane's 16 bytes are then 32 k, i.e. two MFMA steps.
template <typename TIn, int ROWS, int PPT, int U, bool PACKED>  // PPT: 16-value pieces of one row per thread
__global__ __launch_bounds__(256) void decode_fused_kernel(const DecodeArgs d) {
  extern __shared__ __attribute__((aligned(16))) uint8_t xlds[];  // [ROWS][kp]
  __shared__ float smax[ROWS][4];
  __shared__ float sscale[ROWS];
  __shared__ int red[4][16][16];
  constexpr bool XBF = sizeof(TIn) == 2;
  constexpr int WPP = XBF ? 8 : 16;  // 32-bit words of one 16-value input piece
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = (n0 + r) < d.n ? (n0 + r) : (d.n - 1);
  const int kp = (d.k + 255) / 256 * 256;
  const int pieces = d.k / 16;

  constexpr int KS = PACKED ? 128 : 64;   // k covered by one wave-wide weight load
  constexpr int KL = KS / 4;              // k covered by one lane's 16 bytes
  const int kb = PACKED ? d.k / 2 : d.k;  // bytes of one weight row
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, (int64_t)d.n * kb);
  const int kq = ((d.k + 3) / 4 + KS - 1) / KS * KS;
  const int k_lo = wave * kq;
  const int k_hi = (k_lo + kq) < d.k ? (k_lo + kq) : d.k;
  const int wbase = nrow * kb + c * 16;
  auto w_offset = [&](int ko) { return (ko + c * KL < k_hi) ? wbase + (PACKED ? ko / 2 : ko) : kOob; };

  // first batch of weights: in flight while the activations are quantized
  v4i wf[U];
#pragma unroll
  for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(k_lo + u * KS), 0, 0);

  // ---- quantize the activations into LDS
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.x, (int64_t)d.m * d.k * (int64_t)sizeof(TIn));
  uint32_t raw[ROWS][PPT][WPP];
#pragma unroll
  for (int i = 0; i < ROWS; ++i)
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int p = tid + 256 * j;
      const bool ok = i < d.m && p < pieces;
      const int off = ok ? (i * d.k + p * 16) * (int)sizeof(TIn) : kOob;  // out of range reads give 0
#pragma unroll
      for (int q = 0; q < WPP / 4; ++q) {
        const v4i t = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? off + 16 * q : kOob, 0, 0);
        raw[i][j][4 * q + 0] = (uint32_t)t[0]; raw[i][j][4 * q + 1] = (uint32_t)t[1];
        raw[i][j][4 * q + 2] = (uint32_t)t[2]; raw[i][j][4 * q + 3] = (uint32_t)t[3];
      }
    }
  auto value = [&](int i, int j, int e) -> float {
    if constexpr (XBF) {
      const uint32_t w = raw[i][j][e >> 1];
      return __uint_as_float((e & 1) ? (w & 0xFFFF0000u) : (w << 16));
    } else {
      return __uint_as_float(raw[i][j][e]);
    }
  };
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < PPT; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) amax = fmaxf(amax, fabsf(value(i, j, e)));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) smax[i][wave] = amax;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    float amax = fmaxf(fmaxf(smax[i][0], smax[i][1]), fmaxf(smax[i][2], smax[i][3]));
    if (amax == 0.0f) amax = 1.0f;
    float sc = rnd(amax / d.quant_bound, d.x_bf16);
    sc = rnd(sc, d.xs_bf16);
    float inv = rnd(1.0f / sc, d.xs_bf16);
    if (isinf(inv)) inv = 1.0f;
    if (tid == 0) {
      sscale[i] = sc;
      if (blockIdx.x == 0 && i < d.m) d.x_scale_out[i] = sc;
    }
    const int tbf = d.x_bf16 & d.xs_bf16;
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int p = tid + 256 * j;
      uint32_t q[4] = {0u, 0u, 0u, 0u};
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        float t = rnd(value(i, j, e) * inv, tbf);
        t = fminf(fmaxf(t, -d.clip_bound), d.clip_bound);
        q[e >> 2] |= ((uint32_t)((int)rintf(t)) & 0xFFu) << (8 * (e & 3));
      }
      if (p < pieces) {
        const int ps = (p & ~15) | ((p & 15) ^ (i & 15));
        *reinterpret_cast<uint4*>(xlds + (size_t)i * kp + ps * 16) = make_uint4(q[0], q[1], q[2], q[3]);
        if (blockIdx.x == 0 && d.xq_out != nullptr && i < d.m)
          *reinterpret_cast<uint4*>(d.xq_out + (size_t)i * d.k + p * 16) = make_uint4(q[0], q[1], q[2], q[3]);
      }
    }
  }
  __syncthreads();

  // ---- contraction, weights from HBM, activations from LDS
  v4i acc = v4i{0, 0, 0, 0};
  const bool row_ok = r < ROWS && r < d.m;
  constexpr int XP = PACKED ? 2 : 1;  // activation pieces per weight load
  for (int kk = k_lo; kk < k_hi; kk += KS * U) {
    if (kk != k_lo) {
#pragma unroll
      for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(kk + u * KS), 0, 0);
    }
    v4i xf[U][XP];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int h = 0; h < XP; ++h) {
        const int pj = (kk + u * KS) / 16 + c * XP + h;
        xf[u][h] = v4i{0, 0, 0, 0};
        if (row_ok && pj < pieces) {
          const int ps = (pj & ~15) | ((pj & 15) ^ r);
          xf[u][h] = *reinterpret_cast<const v4i*>(xlds + (size_t)r * kp + ps * 16);
        }
      }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if constexpr (PACKED) {
        int t[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) unpack_i4x8((uint32_t)wf[u][j], t[2 * j], t[2 * j + 1]);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][0], v4i{t[0], t[1], t[2], t[3]}, acc, 0, 0, 0);
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][1], v4i{t[4], t[5], t[6], t[7]}, acc, 0, 0, 0);
      } else {
        acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][0], wf[u], acc, 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) red[wave][4 * c + e][r] = acc[e];
  __syncthreads();
  const int mm = tid >> 4, nn = n0 + (tid & 15);
  if (mm < d.m && nn < d.n) {
    const int sum = red[0][mm][tid & 15] + red[1][mm][tid & 15] + red[2][mm][tid & 15] + red[3][mm][tid & 15];
    store_out_scaled(d, mm, nn, sum, sscale[mm]);
  }
}

// ---- packed int4 weights -----------------------------------------------------------------------
// Two int4 per byte, low nibble = even k.  A lane's 16-byte load holds 32 consecutive k of one
// weight row, the B operands of two MFMAs; the matching 32 activation bytes are the two A
// operands.  A nibble is moved to the top of its byte, which makes it 16 * w as a signed int8;
// the factor leaves the accumulator as an exact right shift by 4.  Same workgroup shape as the
// K-split kernel (weights stream from HBM once; half the bytes of the int8 form).

// NB: 16-row weight blocks per wave; every activation fragment a wave loads is used NB times,
// so the L2 traffic for the activations is MB / NB times the int8-equivalent weight bytes.
template <int MB, int NB, int U>  // U: 128-k steps (16 packed bytes per lane and block) in flight per wave
__global__ __launch_bounds__(256) void decode_ksplit_i4_kernel(const DecodeArgs d) {
  __shared__ int red[4][NB][MB * 16][16];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.x * (16 * NB);
  const int kb = d.k / 2;  // bytes of one packed weight row

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, (int64_t)d.n * kb);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.xq, (int64_t)d.m * d.k);
  const int kq = ((d.k + 3) / 4 + 127) / 128 * 128;  // K range of one wave, whole 128-k steps
  const int k_lo = wave * kq;
  const int k_hi = (k_lo + kq) < d.k ? (k_lo + kq) : d.k;
  int wbase[NB], xbase[MB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int row = n0 + nb * 16 + r;
    wbase[nb] = (row < d.n ? row : d.n - 1) * kb + c * 16;  // clamped; such columns are never stored
  }
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) xbase[mb] = (mb * 16 + r) < d.m ? (mb * 16 + r) * d.k + c * 32 : kOob;

  v4i acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = v4i{0, 0, 0, 0};
  for (int kk = k_lo; kk < k_hi; kk += 128 * U) {
    v4i wf[U][NB], xf[U][MB][2];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int ko = kk + u * 128;
      const bool ok = ko + c * 32 < k_hi;  // k is a multiple of 32: a lane's 32 k are all in or all out
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        wf[u][nb] = __builtin_amdgcn_raw_buffer_load_b128(rw, ok ? wbase[nb] + ko / 2 : kOob, 0, 0);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int xo = (ok && xbase[mb] != kOob) ? xbase[mb] + ko : kOob;
        xf[u][mb][0] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo, 0, 0);
        xf[u][mb][1] = __builtin_amdgcn_raw_buffer_load_b128(rx, xo == kOob ? kOob : xo + 16, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        int t[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) unpack_i4x8((uint32_t)wf[u][nb][j], t[2 * j], t[2 * j + 1]);
        const v4i b0 = v4i{t[0], t[1], t[2], t[3]}, b1 = v4i{t[4], t[5], t[6], t[7]};
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][mb][0], b0, acc[mb][nb], 0, 0, 0);
          acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][mb][1], b1, acc[mb][nb], 0, 0, 0);
        }
      }
    __builtin_amdgcn_sched_barrier(0);
  }
  // lane holds C[m = mb*16 + 4c + e][n = n0 + nb*16 + r]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int e = 0; e < 4; ++e) red[wave][nb][mb * 16 + 4 * c + e][r] = acc[mb][nb][e];
  __syncthreads();
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const int mm = mb * 16 + (tid >> 4), nn = n0 + nb * 16 + (tid & 15);
      if (mm < d.m && nn < d.n) {
        const int s = red[0][nb][mm][tid & 15] + red[1][nb][mm][tid & 15] + red[2][nb][mm][tid & 15] +
                      red[3][nb][mm][tid & 15];
        store_out(d, mm, nn, s);
      }
    }
}

// ---- 16 < m <= 64 ------------------------------------------------------------------------------
constexpr int kChunk = 256;  // bytes of K per pipeline step
constexpr int kAhead = 3;    // weight chunks requested ahead of the one being multiplied

// MB: 16-row blocks of activations, 2 (m <= 32) or 4 (m <= 64).  NWV waves own 16 weight rows
// each; KW groups of NWV waves take one K range each (their partial sums meet in LDS at the end),
// which doubles the waves per SIMD for the same weight rows.  K is not split across workgroups.
template <int MB, int NWV, int KW>
__global__ __launch_bounds__(NWV * KW * 64) void decode_block_kernel(const DecodeArgs d) {
  // Activations of one K chunk per K range, [MB*16 rows][256 B]; the 16-byte piece j of row i sits
  // at piece j ^ (i & 15), so the 16 lanes of a fragment read (16 rows, one piece) hit 64 banks.
  __shared__ __attribute__((aligned(16))) uint8_t xbuf[KW][2][MB * 16 * kChunk];
  __shared__ int red[KW > 1 ? (KW - 1) * NWV * MB * 256 : 1];
  constexpr int NT = NWV * 64;           // threads of one K range
  constexpr int XP = MB * 16 * 16 / NT;  // 16-byte pieces of a chunk staged per thread
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int kw = wave / NWV, wn = wave % NWV;
  const int tid = threadIdx.x - kw * NT;  // thread index inside the K range
  const int r = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.x * (NWV * 16) + wn * 16;
  const int nrow = (n0 + r) < d.n ? (n0 + r) : (d.n - 1);  // clamped; such columns are never stored
  const int k_len = ((d.k + KW - 1) / KW + kChunk - 1) / kChunk * kChunk;  // K range, whole chunks
  const int k_lo = kw * k_len;
  const int k_hi = (k_lo + k_len) < d.k ? (k_lo + k_len) : d.k;
  const int nchunks = k_len / kChunk;  // the same for every K range: they share the barriers

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, (int64_t)d.n * d.k);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.xq, (int64_t)d.m * d.k);
  const int wbase = nrow * d.k + c * 16;
  // staging of the activations: thread -> (row tid>>4 of a pass of NT/16 rows, piece tid&15)
  const int xs_row = tid >> 4, xs_piece = tid & 15;

  v4i wreg[kAhead + 1][4], xr[2][XP];  // xr[p]: activations of a chunk of parity p on their way to LDS
  // Workgroups walk the chunks of their K range in rotated order (integer sums do not care):
  // otherwise every workgroup of the launch asks the same few L2 channels for the same
  // activation chunk at the same time.  Step numbers past the range read zeros.
  const int rot = blockIdx.x % nchunks;
  auto chunk_start = [&](int step_no) {
    int j = step_no + rot;
    j = j >= nchunks ? j - nchunks : j;
    return step_no < nchunks ? k_lo + j * kChunk : 0x3FFFFF00;
  };
  auto load_w = [&](v4i* dst, int step_no) {
    const int kc = chunk_start(step_no);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int ko = kc + ks * 64;
      dst[ks] = __builtin_amdgcn_raw_buffer_load_b128(rw, (ko + c * 16 < k_hi) ? wbase + ko : kOob, 0, 0);
    }
  };
  auto load_x = [&](v4i* dst, int step_no) {
    const int kc = chunk_start(step_no);
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int row = p * (NT / 16) + xs_row;
      const int ko = kc + xs_piece * 16;
      dst[p] = __builtin_amdgcn_raw_buffer_load_b128(rx, (row < d.m && ko < k_hi) ? row * d.k + ko : kOob, 0, 0);
    }
  };
  auto store_x = [&](uint8_t* buf, const v4i* src) {
#pragma unroll
    for (int p = 0; p < XP; ++p) {
      const int row = p * (NT / 16) + xs_row;
      *reinterpret_cast<v4i*>(buf + row * kChunk + ((xs_piece ^ (row & 15)) * 16)) = src[p];
    }
  };

  v4i acc[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) acc[mb] = v4i{0, 0, 0, 0};

  load_x(xr[0], 0);
#pragma unroll
  for (int j = 0; j < kAhead; ++j) load_w(wreg[j], j);
  store_x(xbuf[kw][0], xr[0]);
  load_x(xr[1], 1);
  load_x(xr[0], 2);
  __syncthreads();
  // One pipeline step: publish the activations of chunk i+1 (requested two steps ago), request
  // those of chunk i+3 and the weights of chunk i+kAhead, multiply chunk i.  Every load has two
  // or more steps to arrive, so a step never waits a full memory latency.  The register sets
  // rotate roles through the unrolled steps (no register copies that would wait for loads).
  auto step = [&](const v4i* wc, v4i* wfar, v4i* xnext, int i) {
    store_x(xbuf[kw][(i + 1) & 1], xnext);
    load_x(xnext, i + 3);
    load_w(wfar, i + kAhead);
    const uint8_t* buf = xbuf[kw][i & 1];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const v4i xf = *reinterpret_cast<const v4i*>(buf + (mb * 16 + r) * kChunk + (((ks * 4 + c) ^ r) * 16));
        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf, wc[ks], acc[mb], 0, 0, 0);
      }
    // LDS traffic only: a __syncthreads() would also wait for the global loads in flight.
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  static_assert(kAhead == 3, "the unrolled rotation below is written for 4 register sets");
  // Always four steps per trip: steps past the last chunk read zeros everywhere (loads out of
  // range) and add nothing.  A branch-free body lets the compiler count the loads in flight
  // exactly instead of draining them at every loop entry.
  for (int i = 0; i < nchunks; i += 4) {
    step(wreg[0], wreg[3], xr[1], i);
    step(wreg[1], wreg[0], xr[0], i + 1);
    step(wreg[2], wreg[1], xr[1], i + 2);
    step(wreg[3], wreg[2], xr[0], i + 3);
  }

  // lane holds C[m = mb*16 + 4c + e][n = n0 + r]; K ranges 1.. hand their sums to range 0
  if constexpr (KW > 1) {
    if (kw > 0) {
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int e = 0; e < 4; ++e) red[(((kw - 1) * NWV + wn) * MB + mb) * 256 + e * 64 + lane] = acc[mb][e];
    }
    __syncthreads();
    if (kw > 0) return;
#pragma unroll
    for (int j = 1; j < KW; ++j)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int e = 0; e < 4; ++e) acc[mb][e] += red[(((j - 1) * NWV + wn) * MB + mb) * 256 + e * 64 + lane];
  }
  const int nn = n0 + r;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int mm = mb * 16 + 4 * c + e;
      if (mm < d.m && nn < d.n) store_out(d, mm, nn, acc[mb][e]);
    }
}

inline size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

int validate_decode(const aqtx_decode_plan* p) {
  AQTX_REQUIRE(p != nullptr, "aqtx_decode_i8: plan is NULL");
  AQTX_REQUIRE(p->m >= 0 && p->n >= 0 && p->k >= 0, "aqtx_decode_i8: negative shape");
  AQTX_REQUIRE(p->m <= 64, "aqtx_decode_i8: m = %lld exceeds 64 (use aqtx_quantize + aqtx_gemm_i8)",
               (long long)p->m);
  AQTX_REQUIRE(p->w_dtype == AQTX_I8 || p->w_dtype == AQTX_I4 || p->w_dtype == AQTX_I4P,
               "aqtx_decode_i8: w_dtype must be int8, int4 in int8 containers or packed int4");
  const int64_t kmul = p->w_dtype == AQTX_I4P ? 32 : 16;
  AQTX_REQUIRE(p->k > 0 && p->k % kmul == 0, "aqtx_decode_i8: k = %lld must be a positive multiple of %lld",
               (long long)p->k, (long long)kmul);
  AQTX_REQUIRE(p->n * p->k < (1ll << 31) && p->m * p->n < (1ll << 31),
               "aqtx_decode_i8: weight larger than 2 GiB is not addressable with 32-bit offsets");
  AQTX_REQUIRE(is_float_dtype(p->x_dtype) && is_float_dtype(p->x_scale_dtype) &&
                   is_float_dtype(p->w_scale_dtype) && is_float_dtype(p->out_dtype),
               "aqtx_decode_i8: dtypes must be bf16 or f32");
  AQTX_REQUIRE(p->quant_bound > 0.0f && p->clip_bound > 0.0f, "aqtx_decode_i8: bounds must be positive");
  return 0;
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" size_t aqtx_decode_workspace_bytes(const aqtx_decode_plan* p) {
  if (p == nullptr || p->m < 0 || p->n < 0 || p->k < 0 || p->m > 64) return 0;
  return align_up((size_t)(p->m * p->k), 256);  // the quantized activations when the caller keeps none
}

extern "C" int aqtx_decode_i8(const aqtx_decode_plan* p, const void* x, const void* w,
                              const float* w_scale, void* xq, float* x_scale, void* out,
                              void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  if (int rc = validate_decode(p)) return rc;
  if (p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(x != nullptr && w != nullptr && w_scale != nullptr && x_scale != nullptr && out != nullptr,
               "aqtx_decode_i8: NULL buffer");
  const size_t need = xq != nullptr ? 0 : aqtx_decode_workspace_bytes(p);
  AQTX_REQUIRE(need == 0 || (workspace != nullptr && workspace_bytes >= need),
               "aqtx_decode_i8: workspace too small (%zu < %zu)", workspace_bytes, need);
  AQTX_REQUIRE(((uintptr_t)w % 16) == 0 && (need == 0 || ((uintptr_t)workspace % 16) == 0) &&
                   (xq == nullptr || ((uintptr_t)xq % 16) == 0),
               "aqtx_decode_i8: w, xq and the workspace must be 16-byte aligned");
  int8_t* xq_buf = reinterpret_cast<int8_t*>(xq != nullptr ? xq : workspace);
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);

  // 0. a handful of tokens: one kernel quantizes and contracts (AQTX_DECODE_FUSED=0 turns it off)
  {
    const bool xbf = p->x_dtype == AQTX_BF16;
    const int ppt = p->k <= 4096 ? 1 : 2;
    // Every workgroup repeats the quantisation, so its cost grows with the rows while the launch
    // it saves does not: measured at k = 4096, one row gains 2.5 us per call, two rows 1 us,
    // three rows lose.
    const int64_t max_rows = 2;
    const char* fused_env = getenv("AQTX_DECODE_FUSED");
    const bool fused_off = fused_env != nullptr && fused_env[0] == '0';
    if (!fused_off && p->k <= 8192 && p->m <= max_rows && ((uintptr_t)x % 16) == 0) {
      const bool pk = p->w_dtype == AQTX_I4P;
      DecodeArgs d{};
      d.w = reinterpret_cast<const int8_t*>(w);
      d.w_scale = w_scale; d.out = out;
      d.m = (int)p->m; d.n = (int)p->n; d.k = (int)p->k;
      d.out_bf16 = p->out_dtype == AQTX_BF16;
      d.xs_bf16 = p->x_scale_dtype == AQTX_BF16;
      d.ws_bf16 = p->w_scale_dtype == AQTX_BF16;
      d.x = x; d.xq_out = reinterpret_cast<int8_t*>(xq); d.x_scale_out = x_scale;
      d.quant_bound = p->quant_bound; d.clip_bound = p->clip_bound; d.x_bf16 = xbf;
      const unsigned grid = (unsigned)((p->n + 15) / 16);
      const int rows = (int)p->m;
      const size_t lds = (size_t)rows * (size_t)((p->k + 255) / 256 * 256);
      d.acc_shift = pk ? 4 : 0;
#define AQTX_FUSED(T, R, P)                                                   \
  if (pk) decode_fused_kernel<T, R, P, 8, true><<<grid, 256, lds, st>>>(d);  \
  else decode_fused_kernel<T, R, P, 16, false><<<grid, 256, lds, st>>>(d);
      if (xbf) {
        if (ppt == 1) { if (rows == 1) { AQTX_FUSED(uint16_t, 1, 1) } else { AQTX_FUSED(uint16_t, 2, 1) } }
        else { if (rows == 1) { AQTX_FUSED(uint16_t, 1, 2) } else { AQTX_FUSED(uint16_t, 2, 2) } }
      } else {
        if (ppt == 1) { if (rows == 1) { AQTX_FUSED(float, 1, 1) } else { AQTX_FUSED(float, 2, 1) } }
        else { if (rows == 1) { AQTX_FUSED(float, 1, 2) } else { AQTX_FUSED(float, 2, 2) } }
      }
#undef AQTX_FUSED
      AQTX_HIP_CHECK_LAUNCH("decode_fused_kernel");
      return 0;
    }
  }

  // 1. per-token dynamic quantization of the activations (same kernel as training)
  aqtx_quant_plan q{};
  q.in_dtype = q.compute_dtype = p->x_dtype;
  q.scale_dtype = p->x_scale_dtype;
  q.out_dtype = AQTX_I8;
  q.batch = 1; q.rows = p->m; q.cols = p->k;
  q.reduce = AQTX_REDUCE_COLS;
  q.quant_bound = p->quant_bound; q.clip_bound = p->clip_bound;
  q.noise = AQTX_NOISE_NONE;
  if (int rc = aqtx_quantize(&q, x, nullptr, xq_buf, x_scale, nullptr, 0, stream)) return rc;

  // 2. the contraction with the dequantisation fused
  DecodeArgs d{};
  d.xq = xq_buf; d.w = reinterpret_cast<const int8_t*>(w);
  d.x_scale = x_scale; d.w_scale = w_scale; d.out = out;
  d.m = (int)p->m; d.n = (int)p->n; d.k = (int)p->k;
  d.out_bf16 = p->out_dtype == AQTX_BF16;
  d.xs_bf16 = p->x_scale_dtype == AQTX_BF16;
  d.ws_bf16 = p->w_scale_dtype == AQTX_BF16;

  const unsigned grid16 = (unsigned)((p->n + 15) / 16);
  if (p->w_dtype == AQTX_I4P) {
    d.acc_shift = 4;
    const unsigned grid32 = (unsigned)((p->n + 31) / 32);
    // two weight blocks per wave halve the activation re-reads; worth it once n / 32 workgroups
    // still fill the chip
    const bool wide = p->n >= 8192;
    if (p->m <= 16) decode_ksplit_i4_kernel<1, 1, 8><<<grid16, 256, 0, st>>>(d);
    else if (p->m <= 32 && wide) decode_ksplit_i4_kernel<2, 2, 4><<<grid32, 256, 0, st>>>(d);
    else if (p->m <= 32) decode_ksplit_i4_kernel<2, 1, 4><<<grid16, 256, 0, st>>>(d);
    else if (wide) decode_ksplit_i4_kernel<4, 2, 2><<<grid32, 256, 0, st>>>(d);
    else decode_ksplit_i4_kernel<4, 1, 2><<<grid16, 256, 0, st>>>(d);
    AQTX_HIP_CHECK_LAUNCH("decode_ksplit_i4_kernel");
    return 0;
  }
  if (p->m <= 16) {
    decode_ksplit_kernel<1, 16><<<grid16, 256, 0, st>>>(d);
    AQTX_HIP_CHECK_LAUNCH("decode_ksplit_kernel");
    return 0;
  }
  // Whole-K waves sharing the activations through LDS need n/16 >= a few waves per CU to keep
  // HBM busy; below that the K-split shape wins although it re-reads the activations.
  // AQTX_DECODE_SHAPE=ksplit|block overrides the choice (tuning).
  const char* shape_env = getenv("AQTX_DECODE_SHAPE");
  const bool force_ksplit = shape_env != nullptr && shape_env[0] == 'k';
  const bool force_block = shape_env != nullptr && shape_env[0] == 'b';
  if ((p->n < 12288 && !force_block) || force_ksplit) {
    if (p->m <= 32) decode_ksplit_kernel<2, 8><<<grid16, 256, 0, st>>>(d);
    else decode_ksplit_kernel<4, 4><<<grid16, 256, 0, st>>>(d);
    AQTX_HIP_CHECK_LAUNCH("decode_ksplit_kernel");
    return 0;
  }
  const unsigned grid = (unsigned)((p->n + 63) / 64);
  if (p->m <= 32) decode_block_kernel<2, 4, 2><<<grid, 512, 0, st>>>(d);
  else decode_block_kernel<4, 4, 2><<<grid, 512, 0, st>>>(d);
  AQTX_HIP_CHECK_LAUNCH("decode_block_kernel");
  return 0;
}

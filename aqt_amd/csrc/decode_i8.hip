// Serving-shape contraction: out[m, n] = dequant( quant(x)[m, :] . W[n, :] ) for m <= 64 rows of
// activations against a pre-quantized int8 weight stored [n, k] (contraction axis contiguous),
// or an int4 weight packed two values per byte.
//
// The weight is read exactly once and dominates the traffic, so the kernels are built around
// streaming W from HBM with every lane fetching 16 contiguous bytes straight into the operand
// registers of v_mfma_i32_16x16x64_i8 (lane -> row lane&15, bytes 16*(lane>>4).. of a 64-byte
// k step: 16 rows x 64 B per wave instruction, whole 64-byte sectors).
//   m <= 2 : one kernel; every workgroup (16 weight rows) quantizes the activations itself.
//   m >= 3 : a per-token quantize kernel, then a contraction kernel whose workgroups own a tile of
//            weight rows and one K range; partial sums of the K ranges meet through int32 atomics.
#include <type_traits>

#include "common.h"

#include <mutex>

namespace aqtx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef unsigned short dq_u16x2 __attribute__((ext_vector_type(2)));

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
  // K split across workgroups (decode_tile_kernel)
  int k_slice;            // K range of one workgroup (blockIdx.y), a multiple of 4 wave-wide steps
  int splits;             // gridDim.y
  int* sums;              // [n tiles][MB*NB*4][64] int32 exchange words, zero on entry (splits > 1)
  int count_shift;        // bit position of the arrival count inside an exchange word
  // Quantized activations in MFMA fragment order (written by decode_quant_kernel, read by
  // decode_tile_kernel): one 1 KiB block per (K step, 16-token block, half h), holding for lane
  // (r = token in the block, c = k quarter) its 16 operand bytes at c*256 + r*16, so that a
  // wave's fragment load is one contiguous KiB.  A K step is 64 k (int8 weights, one half) or
  // 128 k (packed int4 weights: the lane's 32 k are split in two halves of 16).
  int8_t* xq_frag;
  int mb_total;           // 16-token blocks
  int frag_halves;        // 1 | 2
  // Weight layout.  Rows: [n][k bytes], a wave's load is 16 rows x 64 bytes.  Fragments
  // (aqtx_tile_weight): [16-row block][64-byte k step][1 KiB], the KiB holding for lane
  // (r = row in the block, c = 16-byte quarter) its operand bytes at (c*16 + r)*16, so that a
  // wave's load is one contiguous KiB; rows past n and bytes past the row end are zero.
  int w_frag;             // 1: fragment order
  int w_steps;            // fragment order: 64-byte steps of one row block
  // Activation quantisation inside the contraction launch (decode_tile_kernel): the first `nprod` workgroups of
  // grid row 0 quantize one token each (quant_token_publish) and count themselves in each of kWaitGroups arrival
  // words.  The other workgroups start their weight stream, wait until the arrival word of their group
  // (workgroup number % kWaitGroups) reaches wait_target (at most wait_ticks of the 100 MHz device clock), and
  // count themselves out in their group's departure word when they are done; the last of a group clears the
  // group's two words.  The words lie 128 bytes apart: read-modify-writes on one line take turns at the memory
  // side, about 10 ns each, which hundreds of workgroups on one word would turn into microseconds.  ctrl[1]
  // collects expired waits.
  int nprod;              // 0: the activations were quantized by decode_quant_kernel before this launch
  int* ctrl;              // kControlBytes, zero on entry and (no wait having expired) on exit
  int wait_target;        // nprod (a test makes it unreachable)
  unsigned wait_ticks;
};

constexpr int kWaitGroups = 16;
constexpr int kLineWords = 32;  // 128 bytes
constexpr size_t kControlBytes = (size_t)(1 + 2 * kWaitGroups) * kLineWords * 4 + 128;  // 4352: a multiple of 256
__device__ __forceinline__ int* wait_flag(int* ctrl, int g) { return ctrl + (1 + 2 * g) * kLineWords; }
__device__ __forceinline__ int* departures(int* ctrl, int g) { return ctrl + (2 + 2 * g) * kLineWords; }

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

// A word of eight packed int4 (low nibble = even k) -> two words of int8 holding 16 * value.
__device__ __forceinline__ void unpack_i4x8(uint32_t w, int& lo, int& hi) {
  const uint32_t ev = (w << 4) & 0xF0F0F0F0u;  // k0 k2 k4 k6
  const uint32_t od = w & 0xF0F0F0F0u;         // k1 k3 k5 k7
  lo = (int)__builtin_amdgcn_perm(od, ev, 0x05010400u);  // k0 k1 k2 k3
  hi = (int)__builtin_amdgcn_perm(od, ev, 0x07030602u);  // k4 k5 k6 k7
}

// Workgroup barrier that orders LDS traffic only: __syncthreads() would also wait for the global loads
// in flight (the weights requested ahead of the quantisation).
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
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
// WFRAG: the weight is in fragment order (compile-time here: the offsets of all U loads of a
// batch are then constants off one base register).
template <typename TIn, int ROWS, int PPT, int U, bool PACKED, bool WFRAG>  // PPT: 16-value pieces of one row per thread
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
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, d.w_frag ? (int64_t)((d.n + 15) / 16) * d.w_steps * 1024 : (int64_t)d.n * kb);
  const int kq = ((d.k + 3) / 4 + KS - 1) / KS * KS;
  const int k_lo = wave * kq;
  const int k_hi = (k_lo + kq) < d.k ? (k_lo + kq) : d.k;
  // byte offset of the lane's 16 bytes of k step 0, and what one k step adds to it
  const int wbase = WFRAG ? (int)blockIdx.x * d.w_steps * 1024 + lane * 16 : nrow * kb + c * 16;
  constexpr int wstep = WFRAG ? 1024 : 64;
  auto w_offset = [&](int ko) { return (ko + c * KL < k_hi) ? wbase + (ko / KS) * wstep : kOob; };

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
  // first batch of weights: in flight while the activations are quantized.  Requested after the
  // activations: loads return in order, so the other way round the quantisation would wait for the weights.
  v4i wf[U];
#pragma unroll
  for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(k_lo + u * KS), 0, WFRAG ? kStreamOnce : 0);
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
      for (int e = 0; e < 16; ++e) amax = absmax_step(amax, value(i, j, e));
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = nanmax(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) smax[i][wave] = amax;
  }
  lds_barrier();
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    float amax = nanmax(nanmax(smax[i][0], smax[i][1]), nanmax(smax[i][2], smax[i][3]));
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
  lds_barrier();

  // ---- contraction, weights from HBM, activations from LDS
  v4i acc = v4i{0, 0, 0, 0};
  const bool row_ok = r < ROWS && r < d.m;
  constexpr int XP = PACKED ? 2 : 1;  // activation pieces per weight load
  for (int kk = k_lo; kk < k_hi; kk += KS * U) {
    if (kk != k_lo) {
#pragma unroll
      for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(kk + u * KS), 0, WFRAG ? kStreamOnce : 0);
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

// ---- a few more rows: the same, on 16 waves --------------------------------------------------------
// Quantizing ROWS rows in every workgroup is vector work (about 8 instructions per value), and a wave
// issues a vector instruction only every ~12 cycles: with the four waves of the kernel above it
// takes longer than the weight stream it is meant to hide under.  Here a workgroup has 16 waves:
// all of them quantize (a row is shared by 256 threads, four rows at a time), waves 0..3 alone
// request the weights (before the quantisation) and contract.  Rows are written to LDS as in the
// kernel above.  k <= 4096 * PPT.  The host uses it for ROWS = 4 only: the work every workgroup
// repeats grows with the rows, the launch it saves does not.
template <typename TIn, int ROWS, int PPT, int U, bool PACKED, bool WFRAG>
__global__ __launch_bounds__(1024) void decode_wide_kernel(const DecodeArgs d) {
  static_assert(ROWS % 4 == 0 && ROWS <= 16, "rows come in fours");
  extern __shared__ __attribute__((aligned(16))) uint8_t xlds[];  // [ROWS][kp]
  __shared__ float smax[ROWS][4];
  __shared__ float sscale[ROWS];
  __shared__ int red[4][16][16];
  constexpr bool XBF = sizeof(TIn) == 2;
  constexpr int WPP = XBF ? 8 : 16;  // 32-bit words of one 16-value input piece
  constexpr int PASSES = ROWS / 4;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool contracts = wave < 4;
  const int r = lane & 15, c = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int nrow = (n0 + r) < d.n ? (n0 + r) : (d.n - 1);
  const int kp = (d.k + 255) / 256 * 256;
  const int pieces = d.k / 16;

  constexpr int KS = PACKED ? 128 : 64;   // k covered by one wave-wide weight load
  constexpr int KL = KS / 4;              // k covered by one lane's 16 bytes
  const int kb = PACKED ? d.k / 2 : d.k;  // bytes of one weight row
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, d.w_frag ? (int64_t)((d.n + 15) / 16) * d.w_steps * 1024 : (int64_t)d.n * kb);
  const int kq = ((d.k + 3) / 4 + KS - 1) / KS * KS;
  const int k_lo = (wave & 3) * kq;
  const int k_hi = (k_lo + kq) < d.k ? (k_lo + kq) : d.k;
  const int wbase = WFRAG ? (int)blockIdx.x * d.w_steps * 1024 + lane * 16 : nrow * kb + c * 16;
  constexpr int wstep = WFRAG ? 1024 : 64;
  auto w_offset = [&](int ko) { return (ko + c * KL < k_hi) ? wbase + (ko / KS) * wstep : kOob; };

  // ---- quantize the activations into LDS: thread t works on row 4 * pass + t / 256, pieces t % 256 + 256 j
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.x, (int64_t)d.m * d.k * (int64_t)sizeof(TIn));
  const int sub = tid >> 8, tt = tid & 255, gw = (tid >> 6) & 3;  // row of the pass, thread and wave inside the row's group
  uint32_t raw[PASSES][PPT][WPP];
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps)
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int i = 4 * ps + sub, p = tt + 256 * j;
      const bool ok = i < d.m && p < pieces;
      const int off = ok ? (i * d.k + p * 16) * (int)sizeof(TIn) : kOob;  // out of range reads give 0
#pragma unroll
      for (int q = 0; q < WPP / 4; ++q) {
        const v4i t = __builtin_amdgcn_raw_buffer_load_b128(rx, ok ? off + 16 * q : kOob, 0, 0);
        raw[ps][j][4 * q + 0] = (uint32_t)t[0]; raw[ps][j][4 * q + 1] = (uint32_t)t[1];
        raw[ps][j][4 * q + 2] = (uint32_t)t[2]; raw[ps][j][4 * q + 3] = (uint32_t)t[3];
      }
    }
  v4i wf[U];
  auto value = [&](int ps, int j, int e) -> float {
    if constexpr (XBF) {
      const uint32_t w = raw[ps][j][e >> 1];
      return __uint_as_float((e & 1) ? (w & 0xFFFF0000u) : (w << 16));
    } else {
      return __uint_as_float(raw[ps][j][e]);
    }
  };
  auto quantize_rows = [&]() {
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps) {
    float amax = 0.0f;
    if constexpr (XBF) {
      // two bf16 magnitudes per word: they order like unsigned integers, NaN patterns above infinity
      uint32_t m2 = 0u;
#pragma unroll
      for (int j = 0; j < PPT; ++j)
#pragma unroll
        for (int q = 0; q < WPP; ++q) {
          const dq_u16x2 a2 = __builtin_bit_cast(dq_u16x2, m2), b2 = __builtin_bit_cast(dq_u16x2, raw[ps][j][q] & 0x7FFF7FFFu);
          m2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a2, b2));
        }
      amax = nanmax(__uint_as_float(m2 << 16), __uint_as_float(m2 & 0xFFFF0000u));
    } else {
#pragma unroll
      for (int j = 0; j < PPT; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) amax = absmax_step(amax, value(ps, j, e));
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) amax = nanmax(amax, __shfl_xor(amax, off, 64));
    if (lane == 0) smax[4 * ps + sub][gw] = amax;
  }
  lds_barrier();
  const int tbf = d.x_bf16 & d.xs_bf16;
#pragma unroll
  for (int ps = 0; ps < PASSES; ++ps) {
    const int i = 4 * ps + sub;
    float amax = nanmax(nanmax(smax[i][0], smax[i][1]), nanmax(smax[i][2], smax[i][3]));
    if (amax == 0.0f) amax = 1.0f;
    float sc = rnd(amax / d.quant_bound, d.x_bf16);
    sc = rnd(sc, d.xs_bf16);
    float inv = rnd(1.0f / sc, d.xs_bf16);
    if (isinf(inv)) inv = 1.0f;
    if (tt == 0) {
      sscale[i] = sc;
      if (blockIdx.x == 0 && i < d.m) d.x_scale_out[i] = sc;
    }
    auto quantize_row = [&](auto tbf_c) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int p = tt + 256 * j;
      uint32_t q[4];
#pragma unroll
      for (int w4 = 0; w4 < 4; ++w4) {
        uint32_t b[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float t = value(ps, j, 4 * w4 + e) * inv;
          if constexpr (decltype(tbf_c)::value) t = round_bf16(t);
          // clip, then round half to even and convert in one addition: after t + 1.5 * 2^23 the low
          // mantissa bits are the two's complement of the rounded integer (|t| <= 127 here)
          t = __builtin_amdgcn_fmed3f(t, -d.clip_bound, d.clip_bound);
          b[e] = __float_as_uint(t + 12582912.0f);
        }
        const uint32_t lo = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u);   // bytes b0 b1 0 0
        const uint32_t hi = __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);   // bytes 0 0 b2 b3
        q[w4] = lo | hi;
      }
      if (p < pieces) {
        const int pos = (p & ~15) | ((p & 15) ^ (i & 15));
        *reinterpret_cast<uint4*>(xlds + (size_t)i * kp + pos * 16) = make_uint4(q[0], q[1], q[2], q[3]);
        if (blockIdx.x == 0 && d.xq_out != nullptr && i < d.m)
          *reinterpret_cast<uint4*>(d.xq_out + (size_t)i * d.k + p * 16) = make_uint4(q[0], q[1], q[2], q[3]);
      }
    }
    };
    if (tbf) quantize_row(std::true_type{}); else quantize_row(std::false_type{});
  }
  };
  // The waves that contract request their first batch of weights now, after the activations (loads
  // return in order: the other way round the quantisation would wait for the weights), and quantize
  // with them in flight.  Two copies of the quantisation, one per kind of wave: after a join the
  // compiler would make every wave wait as if it had weights outstanding.
  if (contracts) {
#pragma unroll
    for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(k_lo + u * KS), 0, WFRAG ? kStreamOnce : 0);
    quantize_rows();
  } else {
    quantize_rows();
  }
  lds_barrier();

  // ---- contraction (waves 0..3), weights from HBM, activations from LDS
  if (contracts) {
    v4i acc = v4i{0, 0, 0, 0};
    const bool row_ok = r < ROWS && r < d.m;
    constexpr int XP = PACKED ? 2 : 1;  // activation pieces per weight load
    for (int kk = k_lo; kk < k_hi; kk += KS * U) {
      if (kk != k_lo) {
#pragma unroll
        for (int u = 0; u < U; ++u) wf[u] = __builtin_amdgcn_raw_buffer_load_b128(rw, w_offset(kk + u * KS), 0, WFRAG ? kStreamOnce : 0);
      }
      // four weight loads' worth of activation fragments at a time (all U at once would double the registers)
      constexpr int UC = U < 4 ? U : 4;
#pragma unroll
      for (int u0 = 0; u0 < U; u0 += UC) {
        v4i xf[UC][XP];
#pragma unroll
        for (int u = 0; u < UC; ++u)
#pragma unroll
          for (int h = 0; h < XP; ++h) {
            const int pj = (kk + (u0 + u) * KS) / 16 + c * XP + h;
            xf[u][h] = v4i{0, 0, 0, 0};
            if (row_ok && pj < pieces) {
              const int pos = (pj & ~15) | ((pj & 15) ^ r);
              xf[u][h] = *reinterpret_cast<const v4i*>(xlds + (size_t)r * kp + pos * 16);
            }
          }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < UC; ++u) {
          if constexpr (PACKED) {
            int t[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) unpack_i4x8((uint32_t)wf[u0 + u][j], t[2 * j], t[2 * j + 1]);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][0], v4i{t[0], t[1], t[2], t[3]}, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][1], v4i{t[4], t[5], t[6], t[7]}, acc, 0, 0, 0);
          } else {
            acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(xf[u][0], wf[u0 + u], acc, 0, 0, 0);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) red[wave][4 * c + e][r] = acc[e];
  }
  __syncthreads();
  const int mm = tid >> 4, nn = n0 + (tid & 15);
  if (tid < 256 && mm < d.m && nn < d.n) {
    const int sum = red[0][mm][tid & 15] + red[1][mm][tid & 15] + red[2][mm][tid & 15] + red[3][mm][tid & 15];
    store_out_scaled(d, mm, nn, sum, sscale[mm]);
  }
}

// ---- 3 <= m <= 64: K split across workgroups -----------------------------------------------------
// Phase 1, one workgroup per token: per-token abs-max, scale and int8 values (the arithmetic of the
// row kernel of aqtx_quantize), the row kept in registers between the two passes (PPT 16-value
// pieces per thread; PPT = 0 reads the row twice, any length).  The int8 values are written in
// MFMA fragment order for the contraction kernel (and in plain [m][k] order when the caller asks
// for them); token rows that only pad the last 16-token block are written as zeros.  Every
// workgroup of the launch also clears its share of the exchange words the contraction kernel
// accumulates into, so that no separate clearing launch is needed.
template <typename TIn, int PPT>
__global__ __launch_bounds__(256) void decode_quant_kernel(const DecodeArgs d, uint4* clear, int clear_vec16) {
  __shared__ float smax[4];
  constexpr bool XBF = sizeof(TIn) == 2;
  constexpr int WPP = XBF ? 8 : 16;  // 32-bit words of one 16-value input piece
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int i = blockIdx.x * 256 + tid; i < clear_vec16; i += gridDim.x * 256) clear[i] = make_uint4(0u, 0u, 0u, 0u);
  const int row = blockIdx.x;
  if (row >= d.mb_total * 16) return;  // uniform across the workgroup
  const int pieces = d.k / 16;
  // piece p of this row inside the fragment-ordered copy
  auto frag_ptr = [&](int p) {
    const int step = d.frag_halves == 2 ? p >> 3 : p >> 2;
    const int c = d.frag_halves == 2 ? (p & 7) >> 1 : p & 3;
    const int h = d.frag_halves == 2 ? p & 1 : 0;
    return d.xq_frag + ((int64_t)(step * d.mb_total + (row >> 4)) * d.frag_halves + h) * 1024 + c * 256 + (row & 15) * 16;
  };
  if (row >= d.m) {
    for (int p = tid; p < pieces; p += 256) *reinterpret_cast<uint4*>(frag_ptr(p)) = make_uint4(0u, 0u, 0u, 0u);
    return;
  }
  const TIn* xr = reinterpret_cast<const TIn*>(d.x) + (int64_t)row * d.k;
  constexpr int NP = PPT > 0 ? PPT : 1;
  uint32_t raw[NP][WPP];
  auto load_piece = [&](int p, uint32_t* dst) {
#pragma unroll
    for (int q = 0; q < WPP / 4; ++q) {
      const uint4 t = *reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(xr) + ((int64_t)p * WPP + 4 * q) * 4);
      dst[4 * q + 0] = t.x; dst[4 * q + 1] = t.y; dst[4 * q + 2] = t.z; dst[4 * q + 3] = t.w;
    }
  };
  auto value = [&](const uint32_t* w, int e) -> float {
    if constexpr (XBF) return __uint_as_float((e & 1) ? (w[e >> 1] & 0xFFFF0000u) : (w[e >> 1] << 16));
    else return __uint_as_float(w[e]);
  };
  float amax = 0.0f;
  if constexpr (PPT > 0) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) {
        load_piece(p, raw[j]);
#pragma unroll
        for (int e = 0; e < 16; ++e) amax = absmax_step(amax, value(raw[j], e));
      }
    }
  } else {
    for (int p = tid; p < pieces; p += 256) {
      load_piece(p, raw[0]);
#pragma unroll
      for (int e = 0; e < 16; ++e) amax = absmax_step(amax, value(raw[0], e));
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = nanmax(amax, __shfl_xor(amax, off, 64));
  if (lane == 0) smax[wave] = amax;
  __syncthreads();
  amax = nanmax(nanmax(smax[0], smax[1]), nanmax(smax[2], smax[3]));
  if (amax == 0.0f) amax = 1.0f;
  float sc = rnd(amax / d.quant_bound, d.x_bf16);
  sc = rnd(sc, d.xs_bf16);
  float inv = rnd(1.0f / sc, d.xs_bf16);
  if (isinf(inv)) inv = 1.0f;
  if (tid == 0) d.x_scale_out[row] = sc;
  const int tbf = d.x_bf16 & d.xs_bf16;
  auto quant_piece = [&](const uint32_t* w, int p) {
    uint32_t q[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      float t = rnd(value(w, e) * inv, tbf);
      t = fminf(fmaxf(t, -d.clip_bound), d.clip_bound);
      q[e >> 2] |= ((uint32_t)((int)rintf(t)) & 0xFFu) << (8 * (e & 3));
    }
    const uint4 v = make_uint4(q[0], q[1], q[2], q[3]);
    *reinterpret_cast<uint4*>(frag_ptr(p)) = v;
    if (d.xq_out != nullptr) *reinterpret_cast<uint4*>(d.xq_out + (int64_t)row * d.k + (int64_t)p * 16) = v;
  };
  if constexpr (PPT > 0) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) quant_piece(raw[j], p);
    }
  } else {
    for (int p = tid; p < pieces; p += 256) {
      load_piece(p, raw[0]);
      quant_piece(raw[0], p);
    }
  }
}

// Quantisation of token `row` by one workgroup inside the contraction launch.  The arithmetic is that of decode_quant_kernel: scale = dtype(absmax / bound),
// inv = dtype(1 / scale), q = rint(clip(dtype(x * inv))) (clip with one v_med3, round to nearest even and
// convert with one addition of 1.5 * 2^23: |t| <= 127 there).  The int8 values go to the fragment-ordered copy.
// The workgroups that read them run on other XCDs, whose L2s this one's stores do not reach on their own: scale
// and fragments leave with device scope (written through to memory), the workgroup waits until all of them are
// complete, and only then counts itself in the readers' arrival words with device-scope read-modify-writes.
// Readers touch the copy only after they have seen every producer counted, so no L2 can hold a line of it from
// before.  Up to two 16-value pieces per thread stay in registers between the passes; longer rows are read twice.
__device__ __forceinline__ void quant_token_publish(const DecodeArgs& d, const int row) {
  __shared__ float smax[4];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pieces = d.k / 16;
  const int pw = d.x_bf16 ? 8 : 16;  // 32-bit words of one 16-value input piece
  const uint8_t* xr = reinterpret_cast<const uint8_t*>(d.x) + (int64_t)row * d.k * (d.x_bf16 ? 2 : 4);
  const __amdgpu_buffer_rsrc_t rf = make_rsrc(d.xq_frag, (int64_t)((d.k + 127) / 128) * 2 * d.mb_total * 1024);
  auto frag_off = [&](int p) __attribute__((always_inline)) {
    const int step = d.frag_halves == 2 ? p >> 3 : p >> 2;
    const int c = d.frag_halves == 2 ? (p & 7) >> 1 : p & 3;
    const int h = d.frag_halves == 2 ? p & 1 : 0;
    return (((step * d.mb_total + (row >> 4)) * d.frag_halves + h) << 10) + c * 256 + (row & 15) * 16;
  };
  auto load_piece = [&](int p, uint32_t* dst) __attribute__((always_inline)) {
    const uint4 t0 = *reinterpret_cast<const uint4*>(xr + (int64_t)p * pw * 4);
    const uint4 t1 = *reinterpret_cast<const uint4*>(xr + (int64_t)p * pw * 4 + 16);
    dst[0] = t0.x; dst[1] = t0.y; dst[2] = t0.z; dst[3] = t0.w; dst[4] = t1.x; dst[5] = t1.y; dst[6] = t1.z; dst[7] = t1.w;
    if (!d.x_bf16) {
      const uint4 t2 = *reinterpret_cast<const uint4*>(xr + (int64_t)p * pw * 4 + 32);
      const uint4 t3 = *reinterpret_cast<const uint4*>(xr + (int64_t)p * pw * 4 + 48);
      dst[8] = t2.x; dst[9] = t2.y; dst[10] = t2.z; dst[11] = t2.w; dst[12] = t3.x; dst[13] = t3.y; dst[14] = t3.z; dst[15] = t3.w;
    }
  };
  auto piece_absmax = [&](const uint32_t* w, float amax) __attribute__((always_inline)) -> float {
    if (d.x_bf16) {
      // two bf16 magnitudes per word: they order like unsigned integers, NaN patterns above infinity
      uint32_t m2 = 0u;
#pragma unroll
      for (int q = 0; q < 8; ++q) {
        const dq_u16x2 a2 = __builtin_bit_cast(dq_u16x2, m2), b2 = __builtin_bit_cast(dq_u16x2, w[q] & 0x7FFF7FFFu);
        m2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a2, b2));
      }
      return nanmax(amax, nanmax(__uint_as_float(m2 << 16), __uint_as_float(m2 & 0xFFFF0000u)));
    }
#pragma unroll
    for (int e = 0; e < 16; ++e) amax = absmax_step(amax, __uint_as_float(w[e]));
    return amax;
  };
  const bool held = pieces <= 512;
  uint32_t raw[2][16];
  float amax = 0.0f;
  if (held) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) {
        load_piece(p, raw[j]);
        amax = piece_absmax(raw[j], amax);
      }
    }
  } else {
    for (int p = tid; p < pieces; p += 256) {
      load_piece(p, raw[0]);
      amax = piece_absmax(raw[0], amax);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = nanmax(amax, __shfl_xor(amax, off, 64));
  if (lane == 0) smax[wave] = amax;
  __syncthreads();
  amax = nanmax(nanmax(smax[0], smax[1]), nanmax(smax[2], smax[3]));
  if (amax == 0.0f) amax = 1.0f;
  float sc = rnd(amax / d.quant_bound, d.x_bf16);
  sc = rnd(sc, d.xs_bf16);
  float inv = rnd(1.0f / sc, d.xs_bf16);
  if (isinf(inv)) inv = 1.0f;
  if (tid == 0) __hip_atomic_store(d.x_scale_out + row, sc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const int tbf = d.x_bf16 & d.xs_bf16;
  constexpr int kDeviceScope = 16;  // the sc1 bit of the store's cache policy: written through to memory
  // a whole piece: sixteen values, one 16-byte store
  auto quant_piece = [&](const uint32_t* w, int p) __attribute__((always_inline)) {
    uint32_t q[4];
#pragma unroll
    for (int w4 = 0; w4 < 4; ++w4) {
      uint32_t b[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = 4 * w4 + e;
        const float v = d.x_bf16 ? __uint_as_float((i & 1) ? (w[i >> 1] & 0xFFFF0000u) : (w[i >> 1] << 16)) : __uint_as_float(w[i]);
        float t = rnd(v * inv, tbf);
        t = __builtin_amdgcn_fmed3f(t, -d.clip_bound, d.clip_bound);
        b[e] = __float_as_uint(t + 12582912.0f);
      }
      q[w4] = __builtin_amdgcn_perm(b[1], b[0], 0x0c0c0400u) | __builtin_amdgcn_perm(b[3], b[2], 0x04000c0cu);
    }
    __builtin_amdgcn_raw_buffer_store_b128(v4i{(int)q[0], (int)q[1], (int)q[2], (int)q[3]}, rf, frag_off(p), 0, kDeviceScope);
    if (d.xq_out != nullptr)
      *reinterpret_cast<uint4*>(d.xq_out + (int64_t)row * d.k + (int64_t)p * 16) = make_uint4(q[0], q[1], q[2], q[3]);
  };
  if (held) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int p = tid + 256 * j;
      if (p < pieces) quant_piece(raw[j], p);
    }
  } else {
    for (int p = tid; p < pieces; p += 256) {
      load_piece(p, raw[0]);
      quant_piece(raw[0], p);
    }
  }
  // every store of every thread complete (vmcnt counts stores too on this target), then the count
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  // one count per group of waiting workgroups, lane g the count of group g (nothing comes back: the lanes'
  // additions travel together); only groups that have a member: a count nobody waits for would have nobody to clear it
  const int waiting = ((int)gridDim.x - d.nprod) * (int)gridDim.y;
  if (tid < kWaitGroups && tid < waiting)
    __hip_atomic_fetch_add(wait_flag(d.ctrl, tid), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Phase 2.  A workgroup owns 16*NB weight rows, all m <= 16*MB tokens and one K range
// (blockIdx.y); its four waves take a quarter of that range each.  A wave streams its weight
// fragments from HBM and its activation fragments (fragment order, contiguous KiB) from L2
// straight into MFMA operand registers: every weight fragment meets MB activation fragments and
// every activation fragment NB weight fragments, so the L2 traffic for the activations is
// MB / NB times the weight bytes.  D k-steps are in flight per wave at any time (a ring of
// register sets: the loads of step i + D are issued as soon as step i has been multiplied).
// The weights are the MFMA's row operand, so a lane ends up with four consecutive output
// columns of one token.  The four waves' accumulators meet in LDS.
//
// With one K range per weight tile the workgroup dequantizes and stores.  With several, every
// thread adds its sums to the tile's exchange words with one int32 atomic each (integer addition
// is exact in any order).  The same addition counts the arrival: the addend is
// (1 << count_shift) + sum, and |sum of any subset of the K ranges| < 2^(count_shift - 1), so the
// value the atomic returns says how many K ranges had been added before.  The thread that finds
// every other range already there holds the total (returned value + its own) and dequantizes
// that element.  Device-scope atomic read-modify-writes are carried out at the memory side of the
// per-XCD L2s, so the exchange needs no fence, no second round trip and no waiting loop.
// PACKED: int4 weights two per byte; a lane's 16 bytes are 32 k = two MFMA steps.
//
// With d.nprod the launch quantizes the activations itself (DecodeArgs::nprod): the first nprod workgroups are
// producers and leave after quant_token_publish; the others request their first D steps of weights, wait for
// the producers' count behind a bounded loop (one wave polls with a device-scope read-modify-write, the
// workgroup leaves with ctrl[2] set if the wait expires: every wave reaches its end whatever happens to a
// producer), and only then ask for scales and activation fragments.  The producers have the lowest workgroup
// ids, so they are resident before any workgroup that waits for them.
// DX: K steps of activation fragments in flight per wave (D: of weights).  DX < D is for the launches with
// producers: the weights of D steps are requested before the wait and are there when it ends, the activations
// come from the L2 afterwards and need little in flight; loads return in the order they were requested, so in
// the steady state a wave never has more than DX steps of weights outstanding behind a fragment it waits for.
// PROD: the launch has producers (d.nprod > 0); a template parameter, so that the launches without them keep the
// registers and the instruction stream they had before producers existed.
template <int MB, int NB, int D, bool PACKED, int DX = D, bool PROD = false>
__global__ __launch_bounds__(256, (D * NB * 4 + DX * MB * (PACKED ? 2 : 1) * 4 + MB * NB * 4 + 48 > 256) ? 1 : 2)
void decode_tile_kernel(const DecodeArgs d) {
  static_assert(D % DX == 0, "the fragment ring divides the weight ring");
  constexpr int T = MB * NB;
  constexpr int TPW = (T + 3) / 4;  // 16x16 tiles a wave owns after the reduction: t = wave + 4*j < T
  __shared__ v4i red[4][T][64];
  __shared__ int tokens_ready;
  int bx = (int)blockIdx.x;
  if constexpr (PROD) {
    if (bx < d.nprod) {
      if (blockIdx.y == 0) quant_token_publish(d, bx);
      return;
    }
    bx -= d.nprod;
  }
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  constexpr int KS = PACKED ? 128 : 64;  // k covered by one wave-wide weight load
  constexpr int KL = KS / 4;             // k covered by one lane's 16 bytes
  constexpr int XP = PACKED ? 2 : 1;     // activation fragments per weight fragment
  const int n0 = bx * (16 * NB);
  const int kb = PACKED ? d.k / 2 : d.k;  // bytes of one weight row
  const int s_lo = blockIdx.y * d.k_slice;
  const int s_hi = (s_lo + d.k_slice) < d.k ? (s_lo + d.k_slice) : d.k;
  const int kq = d.k_slice / 4;
  const int k_lo = s_lo + wave * kq;
  const int k_hi = (k_lo + kq) < s_hi ? (k_lo + kq) : s_hi;

  const __amdgpu_buffer_rsrc_t rw = make_rsrc(d.w, d.w_frag ? (int64_t)((d.n + 15) / 16) * d.w_steps * 1024 : (int64_t)d.n * kb);
  const __amdgpu_buffer_rsrc_t rx = make_rsrc(d.xq_frag, (int64_t)((d.k + KS - 1) / KS) * d.mb_total * XP * 1024);
  int wbase[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int row = n0 + nb * 16 + r;
    wbase[nb] = d.w_frag ? (int)(bx * NB + nb) * d.w_steps * 1024 + lane * 16  // past n: reads zeros
                         : (row < d.n ? row : d.n - 1) * kb + c * 16;  // clamped; such columns are never stored
  }

  v4i acc[MB][NB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) acc[mb][nb] = v4i{0, 0, 0, 0};

  // The scales of the outputs this thread will dequantize at the end (tiles t = wave + 4*j: weight
  // block t % NB is the same for all of them), requested now so that they are long there by then.
  float ws[4], xs[TPW];
  {
    const int nn = n0 + (wave % NB) * 16 + 4 * c;  // (wave + 4*j) % NB == wave % NB: NB divides 4
#pragma unroll
    for (int e = 0; e < 4; ++e) ws[e] = d.w_scale[(nn + e) < d.n ? (nn + e) : (d.n - 1)];
  }
  auto load_token_scales = [&]() {
#pragma unroll
    for (int j = 0; j < TPW; ++j) {
      const int mm = ((wave + 4 * j) / NB) * 16 + r;
      xs[j] = d.x_scale[mm < d.m ? mm : (d.m - 1)];
    }
  };
  if constexpr (!PROD) load_token_scales();  // otherwise behind the wait: the producers write them

  const unsigned wstep = d.w_frag ? 1024u : 64u;
  v4i wf[D][NB], xf[DX][MB][XP];
  // Steps past the end of the wave's range, lanes past the end of K and token blocks past m read
  // zeros: their offsets get the out-of-range bits ORed in (no memory access; no branch, which
  // would make the compiler drain the loads in flight).
  // (with producers nobody writes the rows that pad the last 16-token block: their lanes read zeros too)
  unsigned xdead[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) xdead[mb] = (PROD ? mb * 16 + r < d.m : mb < d.mb_total) ? 0u : (unsigned)kOob;
  auto issue_w = [&](auto stream_c, int slot, int ko) {
    constexpr int kPolicy = decltype(stream_c)::value ? kStreamOnce : 0;
    const unsigned dead = (ko + c * KL < k_hi) ? 0u : (unsigned)kOob;  // a lane's KL values are all inside or all outside
    const unsigned wk = (unsigned)(ko / KS) * wstep;  // a k step is 64 bytes of a row, or one KiB fragment
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
      wf[slot][nb] = __builtin_amdgcn_raw_buffer_load_b128(rw, (int)(((unsigned)wbase[nb] + wk) | dead), 0, kPolicy);
  };
  auto issue_x = [&](int slot, int ko) {
    const unsigned dead = (ko + c * KL < k_hi) ? 0u : (unsigned)kOob;
    const unsigned xstep = (unsigned)(ko / KS) * (unsigned)d.mb_total;
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
      for (int h = 0; h < XP; ++h)
        xf[slot][mb][h] = __builtin_amdgcn_raw_buffer_load_b128(
            rx, (int)(((((xstep + mb) * XP + h) << 10) + (unsigned)lane * 16u) | dead | xdead[mb]), 0, 0);
  };
  auto issue = [&](auto stream_c, int slot, int ko) {
    issue_w(stream_c, slot, ko);
    issue_x(slot, ko);
  };
  // The bounded wait for the producers (see the kernel's header).  Returns whether the tokens are there.
  const int wg_id = bx + (int)blockIdx.y * ((int)gridDim.x - d.nprod);
  const int wgroup = wg_id % kWaitGroups;
  auto wait_for_tokens = [&]() -> bool {
    if (wave == 0) {
      const unsigned long long t0 = wall_clock64();
      int flag = 0;
      for (;;) {
        if (lane == 0) flag = __hip_atomic_load(wait_flag(d.ctrl, wgroup), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        flag = __builtin_amdgcn_readfirstlane(flag);
        if (flag >= d.wait_target || wall_clock64() - t0 > d.wait_ticks) break;
        __builtin_amdgcn_s_sleep(2);
      }
      if (lane == 0) {
        if (flag < d.wait_target) __hip_atomic_fetch_or(d.ctrl + 1, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        tokens_ready = flag >= d.wait_target ? 1 : 0;
      }
    }
    lds_barrier();
    return tokens_ready != 0;
  };
  // Counted out of the group; the last one out clears the group's words for the next call.  The count is asked
  // for when the contraction is done and looked at after the outputs have left: nothing waits for it.
  int left_before = 0;
  auto depart = [&]() {
    if (PROD && tid == 0)
      left_before = __hip_atomic_fetch_add(departures(d.ctrl, wgroup), 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };
  auto departed = [&]() {
    const int total = ((int)gridDim.x - d.nprod) * (int)gridDim.y;
    if (PROD && tid == 0 && left_before == (total - wgroup + kWaitGroups - 1) / kWaitGroups - 1) {
      __hip_atomic_fetch_and(wait_flag(d.ctrl, wgroup), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_fetch_and(departures(d.ctrl, wgroup), 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  };
  auto multiply = [&](int slot, int xslot) {
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      if constexpr (PACKED) {
        int t[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) unpack_i4x8((uint32_t)wf[slot][nb][j], t[2 * j], t[2 * j + 1]);
        const v4i b0 = v4i{t[0], t[1], t[2], t[3]}, b1 = v4i{t[4], t[5], t[6], t[7]};
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b0, xf[xslot][mb][0], acc[mb][nb], 0, 0, 0);
          acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(b1, xf[xslot][mb][XP - 1], acc[mb][nb], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
          acc[mb][nb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(wf[slot][nb], xf[xslot][mb][0], acc[mb][nb], 0, 0, 0);
      }
    }
  };
  // Workgroups walk the steps of their K range in rotated order (integer sums do not care):
  // otherwise every workgroup of the launch asks the same L2 channel for the same activation
  // bytes at the same time.  Workgroup ids are dealt round-robin to the 8 XCDs, so id / 8
  // spreads the workgroups that share an L2 evenly over the steps.
  const int nsteps = kq / KS;
  const int rot = (int)(((unsigned)bx / 8 + blockIdx.y) % (unsigned)nsteps);
  auto step_k = [&](int i) {
    int j = i + rot;
    j = j >= nsteps ? j - nsteps : j;
    return i < nsteps ? k_lo + j * KS : 0x3FFFFF00;
  };
  // The weight loads carry the streaming hint when a wave load is a whole KiB fragment; the choice is made
  // once, outside the loop (a branch around a load would make the compiler drain the loads in flight).
  auto walk = [&](auto stream_c) -> bool {
    if constexpr (PROD) {
#pragma unroll
      for (int s = 0; s < D; ++s) issue_w(stream_c, s, step_k(s));
      __builtin_amdgcn_sched_barrier(0);
      if (!wait_for_tokens()) return false;
#pragma unroll
      for (int s = 0; s < DX; ++s) issue_x(s, step_k(s));
      load_token_scales();  // behind the fragments: loads return in order, and these come from further away
    } else if constexpr (DX == D) {
#pragma unroll
      for (int s = 0; s < D; ++s) issue(stream_c, s, step_k(s));
    } else {
#pragma unroll
      for (int s = 0; s < D; ++s) issue_w(stream_c, s, step_k(s));
#pragma unroll
      for (int s = 0; s < DX; ++s) issue_x(s, step_k(s));
    }
    __builtin_amdgcn_sched_barrier(0);
    for (int i = 0; i < nsteps; i += D) {
#pragma unroll
      for (int s = 0; s < D; ++s) {
        multiply(s, s % DX);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (DX == D) {
          issue(stream_c, s, step_k(i + D + s));
        } else {
          issue_x(s % DX, step_k(i + DX + s));
          issue_w(stream_c, s, step_k(i + D + s));
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    return true;
  };
  const bool walked = d.w_frag ? walk(std::true_type{}) : walk(std::false_type{});
  depart();
  if (!walked) {  // the wait expired (ctrl[1] says so): nothing is written
    departed();
    return;
  }
  // lane holds C[n = n0 + nb*16 + 4c + e][m = mb*16 + r] in acc[mb][nb][e]
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) red[wave][mb * NB + nb][lane] = acc[mb][nb];
  __syncthreads();
  // thread -> the lane's four words of tiles t = wave + 4*j < T
  int* tile_sums = d.sums + (int64_t)bx * (T * 4 * 64);
  const int one = 1 << d.count_shift, half = one >> 1;
  const bool wide_ok = (d.n % 4) == 0;  // 4 consecutive outputs of a row are then 8 / 16-byte aligned
  const int p1 = d.out_bf16 & d.xs_bf16;
#pragma unroll
  for (int j = 0; j < TPW; ++j) {
    const int t = wave + 4 * j;
    if (T % 4 != 0 && t >= T) break;  // fewer tiles than waves: the other waves are done (uniform per wave)
    v4i total = red[0][t][lane] + red[1][t][lane] + red[2][t][lane] + red[3][t][lane];
    bool last[4] = {true, true, true, true};
    if (d.splits > 1) {
      int before[4];
#pragma unroll
      for (int e = 0; e < 4; ++e)
        before[e] = __hip_atomic_fetch_add(tile_sums + (t * 4 + e) * 64 + lane, one + total[e], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int arrived = (before[e] + half) >> d.count_shift;  // K ranges added before this one
        total[e] += before[e] - arrived * one;
        last[e] = arrived == d.splits - 1;
        // Every K range has been added: the word goes back to zero for the next call.  A
        // read-modify-write like the additions, so that it is carried out at the same place; a
        // store could sit in this XCD's L2 as part of a line whose other words are still changing.
        if (last[e])
          __hip_atomic_fetch_and(tile_sums + (t * 4 + e) * 64 + lane, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    const int mm = (t / NB) * 16 + r, nn = n0 + (t % NB) * 16 + 4 * c;
    // QTensor.dequant: cast the accumulator, multiply by the lhs scale, then the rhs scale, each
    // product in the promoted dtype of its operands, final cast.
    float f[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float v = rnd((float)(total[e] >> d.acc_shift), d.out_bf16);  // exact: a multiple of 16 when shifted
      v = rnd(v * xs[j], p1);
      v = rnd(v * ws[e], p1 & d.ws_bf16);
      f[e] = rnd(v, d.out_bf16);
    }
    const int64_t o = (int64_t)mm * d.n + nn;
    const bool inside = mm < d.m && nn < d.n;
    if (inside && wide_ok && last[0] && last[1] && last[2] && last[3]) {
      if (d.out_bf16) {
        uint2 v;
        v.x = (uint32_t)bf16_bits(f[0]) | ((uint32_t)bf16_bits(f[1]) << 16);
        v.y = (uint32_t)bf16_bits(f[2]) | ((uint32_t)bf16_bits(f[3]) << 16);
        *reinterpret_cast<uint2*>(reinterpret_cast<uint16_t*>(d.out) + o) = v;
      } else {
        *reinterpret_cast<float4*>(reinterpret_cast<float*>(d.out) + o) = make_float4(f[0], f[1], f[2], f[3]);
      }
    } else if (inside) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (last[e] && nn + e < d.n) {
          if (d.out_bf16) reinterpret_cast<uint16_t*>(d.out)[o + e] = bf16_bits(f[e]);
          else reinterpret_cast<float*>(d.out)[o + e] = f[e];
        }
    }
  }
  departed();
}

// Weight rows -> fragment order (see DecodeArgs): thread -> (16-row block, 64-byte k step, lane).
__global__ __launch_bounds__(256) void tile_weight_kernel(const uint8_t* src, uint8_t* dst, int n, int kb, int steps) {
  const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;  // one 16-byte piece each
  const int64_t frag = id >> 6;
  const int lane = (int)(id & 63);
  const int64_t blk = frag / steps;
  const int step = (int)(frag % steps);
  if (blk * 16 >= n) return;
  const int r = lane & 15, c = lane >> 4;
  const int64_t row = blk * 16 + r;
  const int byte = step * 64 + c * 16;
  uint4 v = make_uint4(0u, 0u, 0u, 0u);
  if (row < n && byte < kb) v = *reinterpret_cast<const uint4*>(src + row * kb + byte);
  *reinterpret_cast<uint4*>(dst + id * 16) = v;
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
  AQTX_REQUIRE(p->n * p->k < (1ll << 31) - 64 && p->m * p->n < (1ll << 31),
               "aqtx_decode_i8: weight larger than 2 GiB is not addressable with 32-bit offsets");
  AQTX_REQUIRE(is_float_dtype(p->x_dtype) && is_float_dtype(p->x_scale_dtype) &&
                   is_float_dtype(p->w_scale_dtype) && is_float_dtype(p->out_dtype),
               "aqtx_decode_i8: dtypes must be bf16 or f32");
  AQTX_REQUIRE(p->quant_bound > 0.0f && p->clip_bound > 0.0f, "aqtx_decode_i8: bounds must be positive");
  AQTX_REQUIRE(p->w_layout == AQTX_W_ROWS || p->w_layout == AQTX_W_FRAGMENTS, "aqtx_decode_i8: unknown w_layout %d",
               p->w_layout);
  AQTX_REQUIRE(p->w_layout == AQTX_W_ROWS || (p->n + 15) / 16 * ((p->k + 63) / 64) * 1024 < (1ll << 31) - 64,
               "aqtx_decode_i8: fragment-ordered weight larger than 2 GiB");
  return 0;
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

// ---- launch shape of the split-K path ------------------------------------------------------------
namespace {

struct TileShape {
  int mb, nb, depth;  // template parameters of decode_tile_kernel
  int ntiles;         // weight tiles of 16*nb rows
  int splits;         // K ranges (workgroups per weight tile)
  int k_slice;        // K per range
  int count_shift;    // arrival count position in an exchange word
  size_t sums_bytes;  // exchange words actually used (0 when splits == 1)
};

// plan->tuning, all fields 0 = the library's choice:
//   bits 0-7 K ranges per weight tile, bits 8-11 nb (1 | 2 | 4), bits 12-15 K steps in flight
//   per wave (2 | 4 | 8 | 15 for 16), bits 16-19 path (1 = one or two tokens take the path of three and more)
TileShape choose_tile_shape(const aqtx_decode_plan* p) {
  TileShape t{};
  const int tune = p->tuning;
  const bool packed = p->w_dtype == AQTX_I4P;
  const int ks = packed ? 128 : 64;
  t.mb = p->m <= 16 ? 1 : p->m <= 32 ? 2 : 4;
  // About one workgroup per CU (256): the tallest weight tile (64, 32 or 16 rows) that still gives
  // 192 tiles or more (a taller tile re-reads the activations less often); whatever is then
  // still missing comes from splitting K, which costs exchange traffic in proportion to
  // m * n * K ranges.  Measured at k = 4096: n = 4096 is fastest with 16-row tiles and no split,
  // n = 14336 with 64-row tiles and no split.
  int nb_auto = 4;
  while (nb_auto > 1 && (p->n + 16 * nb_auto - 1) / (16 * nb_auto) < 192) nb_auto /= 2;
  t.nb = ((tune >> 8) & 15) ? ((tune >> 8) & 15) : nb_auto;
  if (t.nb != 1 && t.nb != 2 && t.nb != 4) t.nb = nb_auto;
  t.ntiles = (int)((p->n + 16 * t.nb - 1) / (16 * t.nb));
  // An exchange word holds count * 2^shift + sum with |sum| <= k * 127 * 128 < 2^(shift - 1).
  int magnitude_bits = 1;
  while (((int64_t)1 << magnitude_bits) <= p->k * (int64_t)(127 * 128)) ++magnitude_bits;
  t.count_shift = magnitude_bits + 1;
  const int max_by_count = t.count_shift >= 31 ? 1 : (1 << (31 - t.count_shift)) - 1;
  const int max_by_k = (int)((p->k + 4 * ks - 1) / (4 * ks));  // at least one step per wave
  int splits = tune & 255;
  if (splits == 0) splits = (256 + t.ntiles / 2) / t.ntiles;
  if (splits > max_by_k) splits = max_by_k;
  if (splits > max_by_count) splits = max_by_count;
  if (splits < 1) splits = 1;
  int k_slice = (int)((p->k + splits - 1) / splits);
  k_slice = (k_slice + 4 * ks - 1) / (4 * ks) * (4 * ks);
  t.k_slice = k_slice;
  t.splits = (int)((p->k + k_slice - 1) / k_slice);
  const int steps = k_slice / (4 * ks);
  const int loads_per_step = t.nb + t.mb * (packed ? 2 : 1);
  t.depth = ((tune >> 12) & 15) ? ((tune >> 12) & 15) : ((steps >= 4 && (t.mb == 1 || t.nb == 1)) ? 4 : 2);
  if (t.depth == 15) t.depth = 16;  // the 4-bit field cannot say 16
  if (t.depth != 2 && t.depth != 4 && t.depth != 8 && t.depth != 16) t.depth = 4;
  while (t.depth > 2 && t.depth * loads_per_step > 64) t.depth /= 2;  // 256 registers of operands in flight
  while (t.depth > 2 && t.depth > steps) t.depth /= 2;                // steps past the range are wasted issue slots
  if (t.splits > 1) t.sums_bytes = (size_t)t.ntiles * t.mb * t.nb * 1024;
  return t;
}

// Upper bound of the exchange words over every launch shape: 64 token rows x (n rounded up to a
// whole tile) int32 words.
// Before them, in the first kControlBytes of a workspace, the control words of the launches that quantize the
// activations themselves.
size_t exchange_bytes_bound(const aqtx_decode_plan* p) { return kControlBytes + (size_t)64 * (size_t)(p->n + 64) * 4; }
// The quantized activations in fragment order: 64 token rows x k rounded up to a whole K step.
size_t fragment_bytes_bound(const aqtx_decode_plan* p) { return (size_t)64 * (size_t)((p->k + 127) / 128 * 128) + 256; }

template <bool PACKED>
int launch_tile(const TileShape& t, const DecodeArgs& d, hipStream_t st) {
  const dim3 grid((unsigned)(t.ntiles + d.nprod), (unsigned)t.splits);
#define AQTX_TILE(MB, NB, D) decode_tile_kernel<MB, NB, D, PACKED><<<grid, 256, 0, st>>>(d)
  // depths whose operands in flight fit the register file: (nb + mb * halves) * depth <= 64 loads
#define AQTX_TILE_D(MB, NB)                                                          \
  do {                                                                               \
    constexpr int kLoads = NB + MB * (PACKED ? 2 : 1);                               \
    if constexpr (kLoads * 16 <= 64) { if (t.depth == 16) { AQTX_TILE(MB, NB, 16); break; } } \
    if constexpr (kLoads * 8 <= 64) { if (t.depth >= 8) { AQTX_TILE(MB, NB, 8); break; } }    \
    if (t.depth >= 4 && kLoads * 4 <= 64) { AQTX_TILE(MB, NB, 4); break; }           \
    AQTX_TILE(MB, NB, 2);                                                            \
  } while (0)
#define AQTX_TILE_N(MB)                         \
  do {                                          \
    if (t.nb == 1) AQTX_TILE_D(MB, 1);          \
    else if (t.nb == 2) AQTX_TILE_D(MB, 2);     \
    else AQTX_TILE_D(MB, 4);                    \
  } while (0)
  // With producers: all (or as many as the registers hold) of a wave's weight steps are requested before the
  // wait, few steps of fragments are in flight (see DX): one shape per (mb, nb).
#define AQTX_TILE_P(MB, NB, DW, DXV) \
  decode_tile_kernel<MB, NB, (PACKED ? DW / 2 : DW), PACKED, (PACKED && DXV > 2 ? DXV / 2 : DXV), true><<<grid, 256, 0, st>>>(d)
#define AQTX_TILE_PN(MB, D4, X1, X2, X4)            \
  do {                                              \
    if (t.nb == 1) AQTX_TILE_P(MB, 1, 16, X1);      \
    else if (t.nb == 2) AQTX_TILE_P(MB, 2, 16, X2); \
    else AQTX_TILE_P(MB, 4, D4, X4);                \
  } while (0)
  if (d.nprod) {
    if (t.mb == 1) AQTX_TILE_PN(1, 8, 16, 8, 8);
    else if (t.mb == 2) AQTX_TILE_PN(2, 8, 8, 4, 4);
    else AQTX_TILE_PN(4, 4, 4, 2, 4);
  } else if (t.mb == 1) AQTX_TILE_N(1);
  else if (t.mb == 2) AQTX_TILE_N(2);
  else AQTX_TILE_N(4);
#undef AQTX_TILE_PN
#undef AQTX_TILE_P
#undef AQTX_TILE_N
#undef AQTX_TILE_D
#undef AQTX_TILE
  AQTX_HIP_CHECK_LAUNCH("decode_tile_kernel");
  return 0;
}

template <typename TIn>
int launch_decode_quant(const DecodeArgs& d, uint4* clear, int clear_vec16, hipStream_t st) {
  int clear_blocks = (clear_vec16 + 1023) / 1024;
  if (clear_blocks > 256) clear_blocks = 256;
  const int rows = d.mb_total * 16;
  const unsigned grid = (unsigned)(rows > clear_blocks ? rows : clear_blocks);
  const int pieces = d.k / 16;
  if (pieces <= 256) decode_quant_kernel<TIn, 1><<<grid, 256, 0, st>>>(d, clear, clear_vec16);
  else if (pieces <= 512) decode_quant_kernel<TIn, 2><<<grid, 256, 0, st>>>(d, clear, clear_vec16);
  else if (pieces <= 1024) decode_quant_kernel<TIn, 4><<<grid, 256, 0, st>>>(d, clear, clear_vec16);
  else decode_quant_kernel<TIn, 0><<<grid, 256, 0, st>>>(d, clear, clear_vec16);
  AQTX_HIP_CHECK_LAUNCH("decode_quant_kernel");
  return 0;
}

}  // namespace

extern "C" size_t aqtx_decode_workspace_bytes(const aqtx_decode_plan* p) {
  if (p == nullptr || p->m < 0 || p->n < 0 || p->k < 0 || p->m > 64) return 0;
  // the partial-sum exchange first, then the quantized activations when the caller keeps none
  return exchange_bytes_bound(p) + fragment_bytes_bound(p);
}

extern "C" size_t aqtx_decode_exchange_bytes(const aqtx_decode_plan* p) {
  if (p == nullptr || p->m < 0 || p->n < 0 || p->k < 0 || p->m > 64) return 0;
  return exchange_bytes_bound(p);
}

namespace {

int decode_impl(const aqtx_decode_plan* p, const void* x, const void* w, const float* w_scale, void* xq,
                float* x_scale, void* out, void* workspace, size_t workspace_bytes, void* stream) {
  if (p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(x != nullptr && w != nullptr && w_scale != nullptr && x_scale != nullptr && out != nullptr,
               "aqtx_decode_i8: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)w % 16) == 0 && ((uintptr_t)x % 16) == 0 && (xq == nullptr || ((uintptr_t)xq % 16) == 0),
               "aqtx_decode_i8: x, w and xq must be 16-byte aligned");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  const bool xbf = p->x_dtype == AQTX_BF16;
  const bool pk = p->w_dtype == AQTX_I4P;

  DecodeArgs d{};
  d.w = reinterpret_cast<const int8_t*>(w);
  d.w_scale = w_scale; d.out = out;
  d.m = (int)p->m; d.n = (int)p->n; d.k = (int)p->k;
  d.out_bf16 = p->out_dtype == AQTX_BF16;
  d.xs_bf16 = p->x_scale_dtype == AQTX_BF16;
  d.ws_bf16 = p->w_scale_dtype == AQTX_BF16;
  d.x = x; d.x_scale_out = x_scale;
  d.quant_bound = p->quant_bound; d.clip_bound = p->clip_bound; d.x_bf16 = xbf;
  d.acc_shift = pk ? 4 : 0;
  d.w_frag = p->w_layout == AQTX_W_FRAGMENTS;
  d.w_steps = (int)(((pk ? p->k / 2 : p->k) + 63) / 64);

  // One or two tokens: one kernel quantizes and contracts.  Every workgroup repeats the
  // quantisation, so its cost grows with the rows while the launch it saves does not: measured at
  // k = 4096, one row gains 2.5 us per call, two rows 1 us, three rows lose.
  const bool never_fuse = ((p->tuning >> 16) & 15) != 0;
  if (!never_fuse && p->k <= 8192 && p->m <= 2) {
    d.xq_out = reinterpret_cast<int8_t*>(xq);
    const int ppt = p->k <= 4096 ? 1 : 2;
    const unsigned grid = (unsigned)((p->n + 15) / 16);
    const int rows = (int)p->m;
    const size_t lds = (size_t)rows * (size_t)((p->k + 255) / 256 * 256);
#define AQTX_FUSED(T, R, P)                                                                       \
  if (d.w_frag) {                                                                                 \
    if (pk) decode_fused_kernel<T, R, P, 8, true, true><<<grid, 256, lds, st>>>(d);              \
    else decode_fused_kernel<T, R, P, 16, false, true><<<grid, 256, lds, st>>>(d);               \
  } else {                                                                                        \
    if (pk) decode_fused_kernel<T, R, P, 8, true, false><<<grid, 256, lds, st>>>(d);             \
    else decode_fused_kernel<T, R, P, 16, false, false><<<grid, 256, lds, st>>>(d);              \
  }
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

  // Three or four tokens against a weight of at most 256 16-row blocks (one workgroup per CU, so the
  // quantisation every workgroup repeats is paid once): one kernel again, on 16 waves per workgroup.
  // Measured at k = 4096, n = 4096: 7.7 us against 9.0-9.2 us for the two kernels below; with 8 rows
  // per workgroup the two are equal and with 16 this one loses by 3 us (its time grows by 0.37 us per
  // row, the vector work of quantizing a row on one CU, whatever the weight loads in flight); with
  // several rounds of workgroups (n = 14336) the repeated quantisation loses by 5-12 us.
  const unsigned wide_grid = (unsigned)((p->n + 15) / 16);
  if (!never_fuse && p->m <= 4 && p->k <= 8192 && wide_grid <= 256) {
    d.xq_out = reinterpret_cast<int8_t*>(xq);
    const size_t lds = (size_t)4 * (size_t)((p->k + 255) / 256 * 256);
#define AQTX_WIDE(T, P)                                                                          \
  if (d.w_frag) {                                                                                \
    if (pk) decode_wide_kernel<T, 4, P, 4, true, true><<<wide_grid, 1024, lds, st>>>(d);         \
    else decode_wide_kernel<T, 4, P, 8, false, true><<<wide_grid, 1024, lds, st>>>(d);           \
  } else {                                                                                       \
    if (pk) decode_wide_kernel<T, 4, P, 4, true, false><<<wide_grid, 1024, lds, st>>>(d);        \
    else decode_wide_kernel<T, 4, P, 8, false, false><<<wide_grid, 1024, lds, st>>>(d);          \
  }
    if (xbf) { if (p->k <= 4096) { AQTX_WIDE(uint16_t, 1) } else { AQTX_WIDE(uint16_t, 2) } }
    else { if (p->k <= 4096) { AQTX_WIDE(float, 1) } else { AQTX_WIDE(float, 2) } }
#undef AQTX_WIDE
    AQTX_HIP_CHECK_LAUNCH("decode_wide_kernel");
    return 0;
  }

  const TileShape t = choose_tile_shape(p);
  const size_t exch = t.sums_bytes;
  const size_t need = exchange_bytes_bound(p) + fragment_bytes_bound(p);
  AQTX_REQUIRE(workspace != nullptr && workspace_bytes >= need,
               "aqtx_decode_i8: workspace too small (%zu < %zu)", workspace_bytes, need);
  AQTX_REQUIRE(((uintptr_t)workspace % 256) == 0, "aqtx_decode_i8: the workspace must be 256-byte aligned");
  uint8_t* ws = reinterpret_cast<uint8_t*>(workspace);
  // exchange words at the start, fragments in the last bytes: in a workspace shared by calls of
  // different shapes no call's fragments land on words another call expects to be zero
  const size_t frag_off = (workspace_bytes - fragment_bytes_bound(p)) / 256 * 256;
  d.xq_frag = reinterpret_cast<int8_t*>(ws + frag_off);
  d.mb_total = (int)((p->m + 15) / 16);
  d.frag_halves = pk ? 2 : 1;

  d.xq_out = reinterpret_cast<int8_t*>(xq);
  d.k_slice = t.k_slice; d.splits = t.splits;
  d.sums = reinterpret_cast<int*>(ws + kControlBytes);
  d.count_shift = t.count_shift;

  // One launch: the first workgroups quantize a token each while the others already stream their weights
  // (decode_tile_kernel with producers).  It counts in control words that must be zero on entry, so it is for
  // callers that vouch for their workspace; the others get the two launches below, the first of which clears.
  // Between the start of the launch and the first matrix instruction lie the row's load, the write-through of its
  // int8 values, the count, the poll that sees it and the first fragment load: five trips to memory, about a
  // microsecond each, against two for the weights.  Measured (k = 4096, HIP-graph replay): against the 58.7 MB
  // weight the one launch takes 13.5 / 13.8 / 15.0 us for 8 / 16 / 32 tokens where the two take 15.0 / 15.0 / 15.5
  // (packed int4: 9.9 / 10.4 against 10.4 / 10.6 for 8 / 16); with 64 tokens, or against the 16.8 MB weight, whose
  // stream is over before the chain is, the two launches are as fast or faster (8.5 against 9.2 us at 8 tokens).
  const int path = (p->tuning >> 16) & 15;
  const int64_t w_bytes = p->n * (pk ? p->k / 2 : p->k);
  const bool pays = path == 1 || (w_bytes >= (24ll << 20) && p->m <= (pk ? 16 : 32));
  if (p->workspace_zeroed && path != 2 && pays) {
    // (four producers per token, a quarter of every piece each, measured 0.1-0.4 us slower up to 8 tokens and 2-4 us
    // slower from 32 on, where their workgroups delay the readers' start; so did four workgroups per token in the
    // quantize launch of the two-launch form)
    d.nprod = (int)p->m;
    d.ctrl = reinterpret_cast<int*>(ws);
    const bool expire = ((p->tuning >> 20) & 15) == 1;  // test hook: a count that never comes, a wait of a microsecond
    d.wait_target = expire ? d.nprod + 1 : d.nprod;
    d.wait_ticks = expire ? 100u : 20000000u;  // 0.2 s of the 100 MHz clock
    d.x_scale = x_scale;
    return pk ? launch_tile<true>(t, d, st) : launch_tile<false>(t, d, st);
  }

  // 1. per-token dynamic quantisation of the activations; the same launch clears the exchange
  //    words unless the caller vouches for them
  const int clear16 = p->workspace_zeroed ? 0 : (int)(exch / 16);
  if (int rc = xbf ? launch_decode_quant<uint16_t>(d, reinterpret_cast<uint4*>(d.sums), clear16, st)
                   : launch_decode_quant<float>(d, reinterpret_cast<uint4*>(d.sums), clear16, st))
    return rc;

  // 2. the contraction with the dequantisation fused
  d.x_scale = x_scale;
  return pk ? launch_tile<true>(t, d, st) : launch_tile<false>(t, d, st);
}

// ---- scratch of the entry point that allocates nothing -------------------------------------------
// Room for the exchange words and the fragment-ordered activations of any call with
// n <= kStaticMaxN and k <= kStaticMaxK.  Every GPU the library runs on holds its own copy of the
// array for the life of the process.
constexpr int64_t kStaticMaxN = 32768, kStaticMaxK = 32768;
constexpr size_t kStaticScratchBytes =
    kControlBytes + (size_t)64 * (size_t)(kStaticMaxN + 64) * 4 + (size_t)64 * (size_t)kStaticMaxK + 512;  // 10.6 MB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// Device address of `scratch` on each GPU, looked up once per device (the array's name is only a
// host-side handle: it must never reach a kernel or a memset as a pointer).
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

int static_scratch(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return set_error("aqtx_decode_i8_static: hipGetDevice failed: %s", hipGetErrorString(e));
  AQTX_REQUIRE(dev >= 0 && dev < kMaxDevices, "aqtx_decode_i8_static: device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* sym = nullptr;
    e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
    if (e != hipSuccess || sym == nullptr)
      return set_error("aqtx_decode_i8_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = sym;
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

}  // namespace

extern "C" int aqtx_decode_i8(const aqtx_decode_plan* p, const void* x, const void* w,
                              const float* w_scale, void* xq, float* x_scale, void* out,
                              void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  if (int rc = validate_decode(p)) return rc;
  return decode_impl(p, x, w, w_scale, xq, x_scale, out, workspace, workspace_bytes, stream);
}

extern "C" int aqtx_decode_i8_check(void* workspace, size_t workspace_bytes, void* stream) {
  clear_error();
  AQTX_REQUIRE(workspace != nullptr && workspace_bytes >= kControlBytes, "aqtx_decode_i8_check: workspace too small");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  int* ctrl = reinterpret_cast<int*>(workspace);
  int words[2] = {0, 0};
  hipError_t e = hipMemcpyAsync(words, ctrl, sizeof words, hipMemcpyDeviceToHost, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  if (e != hipSuccess) return set_error("aqtx_decode_i8_check: reading the control words failed: %s", hipGetErrorString(e));
  if (words[1] == 0) return 0;
  e = hipMemsetAsync(ctrl, 0, kControlBytes, st);
  if (e == hipSuccess) e = hipStreamSynchronize(st);
  return set_error("aqtx_decode_i8: a wait for the quantized activations expired in an earlier call on this workspace "
                   "(mark %d); its outputs are incomplete%s", words[1],
                   e == hipSuccess ? "; the control words have been cleared" : "");
}

extern "C" int aqtx_decode_i8_static(const aqtx_decode_plan* p, const void* x, const void* w,
                                     const float* w_scale, void* xq, float* x_scale, void* out,
                                     void* stream) {
  clear_error();
  if (int rc = validate_decode(p)) return rc;
  AQTX_REQUIRE(p->n <= kStaticMaxN && p->k <= kStaticMaxK,
               "aqtx_decode_i8_static: n = %lld, k = %lld exceed the built-in scratch (n <= %lld, k <= %lld); "
               "use aqtx_decode_i8 with a workspace",
               (long long)p->n, (long long)p->k, (long long)kStaticMaxN, (long long)kStaticMaxK);
  if (p->m == 0 || p->n == 0) return 0;
  void* ws = nullptr;
  if (int rc = static_scratch(&ws)) return rc;
  // The array keeps whatever the last call on this GPU left: the exchange words a call uses are
  // cleared by its first kernel, never assumed to be zero.
  aqtx_decode_plan plan = *p;
  plan.workspace_zeroed = 0;
  return decode_impl(&plan, x, w, w_scale, xq, x_scale, out, ws, kStaticScratchBytes, stream);
}

extern "C" size_t aqtx_tile_weight_bytes(int64_t n, int64_t k, int32_t w_dtype) {
  if (n <= 0 || k <= 0) return 0;
  const int64_t kb = w_dtype == AQTX_I4P ? k / 2 : k;
  return (size_t)((n + 15) / 16) * (size_t)((kb + 63) / 64) * 1024;
}

extern "C" int aqtx_tile_weight(const void* src, void* dst, int64_t n, int64_t k, int32_t w_dtype, void* stream) {
  clear_error();
  AQTX_REQUIRE(w_dtype == AQTX_I8 || w_dtype == AQTX_I4 || w_dtype == AQTX_I4P,
               "aqtx_tile_weight: w_dtype must be int8, int4 in int8 containers or packed int4");
  AQTX_REQUIRE(n >= 0 && k >= 0, "aqtx_tile_weight: negative shape");
  const int64_t kmul = w_dtype == AQTX_I4P ? 32 : 16;
  AQTX_REQUIRE(k % kmul == 0, "aqtx_tile_weight: k = %lld must be a multiple of %lld", (long long)k, (long long)kmul);
  if (n == 0 || k == 0) return 0;
  AQTX_REQUIRE(src != nullptr && dst != nullptr, "aqtx_tile_weight: NULL buffer");
  AQTX_REQUIRE(((uintptr_t)src % 16) == 0 && ((uintptr_t)dst % 16) == 0, "aqtx_tile_weight: buffers must be 16-byte aligned");
  const int64_t kb = w_dtype == AQTX_I4P ? k / 2 : k;
  const int64_t steps = (kb + 63) / 64;
  const int64_t pieces = (n + 15) / 16 * steps * 64;
  AQTX_REQUIRE(pieces / 256 + 1 < (1ll << 31), "aqtx_tile_weight: weight too large for one launch");
  tile_weight_kernel<<<dim3((unsigned)((pieces + 255) / 256)), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const uint8_t*>(src), reinterpret_cast<uint8_t*>(dst), (int)n, (int)kb, (int)steps);
  AQTX_HIP_CHECK_LAUNCH("tile_weight_kernel");
  return 0;
}

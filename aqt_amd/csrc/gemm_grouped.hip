// int8 x int8/int4 contraction with one scale pair per group of the contraction axis
// (subchannel / tiled quantization): for every group g of `group` consecutive k,
//   part_g[m, n] = round( round( cast(sum_{k in g} A[m,k] B[n,k]) * s_row[g][m] ) * s_col[g][n] )
//   C[m, n]      = cast( sum_g part_g[m, n] )          (float32 accumulation in group order)
// which is what tiled_dot_general does with a quantizing inner dot_general: the tile-count axis is
// a batch axis of the inner call, every tile is dequantized (rounded to the dequant dtype) on its
// own and the tiles are summed afterwards.  Here the per-group results never leave registers.
//
// One workgroup (8 waves, 2x4) owns a 128x256 tile of C, a wave 64x64 = 2x2 MFMA tiles
// (v_mfma_i32_32x32x32_i8): 64 int32 accumulators of the current group and 64 float32 running
// sums.  A stage is 128 bytes of K, double-buffered in LDS with the same XOR swizzle as the dense
// kernel.  The group scales of a stage sit in LDS next to it.  The per-group rescale is ~9 VALU
// operations per element and group, which bounds this kernel (the MFMAs of one wave run under the
// rescale of the other wave of its SIMD).
//
// Packed int4 weights (two values per byte, low nibble = even k) are unpacked in registers on their
// way to LDS: a nibble is moved to the top of its byte (value * 16) and the factor 1/16 is folded,
// exactly, into the column scale.
#include "gemm_core.h"

namespace aqtx {
namespace {

constexpr int GM = 128, GN = 256;  // GK = BK = 128

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Rounds two floats to bf16 (ties to even) in place: one packed conversion, then one shift and
// one mask to widen them again.
template <bool kBf16>
__device__ __forceinline__ void round_pair(float& a, float& b) {
  if constexpr (kBf16) {
    const bf16x2 h = __builtin_convertvector(f32x2{a, b}, bf16x2);
    const uint32_t w = __builtin_bit_cast(uint32_t, h);
    a = __uint_as_float(w << 16);
    b = __uint_as_float(w & 0xFFFF0000u);
  }
}

struct GroupedArgs {
  const uint8_t* a;        // int8 [m][lda]
  const uint8_t* b;        // int8 [n][ldb], or packed int4 [n][ldb] with ldb in bytes (= k/2)
  const float* row_scale;  // [groups][m]
  const float* col_scale;  // [groups][n]
  void* c;                 // [m][ldc]
  int64_t m, n, k, lda, ldb, ldc;
  int groups, stages_per_group;
  int tiles_m, tiles_n;
};

// EPI as in the dense kernel: 0 = bf16 out, both products rounded to bf16; 4 = bf16 out, first
// product bf16, second f32; 1 = bf16 out, products in f32; 2 = f32 out.
// ONE: a group is exactly one 128-byte stage (group = 128), which takes the branches on the
// position inside a group out of the loop.
template <int EPI, bool PACKED, bool ONE>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_grouped_kernel(const GroupedArgs g) {
  constexpr bool kOutBf16 = EPI != 2;
  constexpr bool kP1Bf16 = EPI == 0 || EPI == 4;
  constexpr bool kP2Bf16 = EPI == 0;
  constexpr int kATile = GM * BK, kBTile = GN * BK, kStage = kATile + kBTile;  // 48 KiB
  __shared__ __attribute__((aligned(1024))) uint8_t stage_mem[2][kStage];
  __shared__ __attribute__((aligned(16))) float srow[2][GM];
  __shared__ __attribute__((aligned(16))) float scol[2][GN];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;
  const int lr = lane & 31, lh = lane >> 5;
  int tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t m0 = (int64_t)tm * GM, n0 = (int64_t)tn * GN;
  const int64_t rows_a = (g.m - m0) < GM ? (g.m - m0) : GM;
  const int64_t rows_b = (g.n - n0) < GN ? (g.n - n0) : GN;
  const int kb_bytes = PACKED ? (int)(g.k / 2) : (int)g.k;  // bytes of one B row
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(g.a + m0 * g.lda), 0, (int)((rows_a - 1) * g.lda + g.k), kBufferRsrcWord3);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(g.b + n0 * g.ldb), 0, (int)((rows_b - 1) * g.ldb + kb_bytes), kBufferRsrcWord3);

  // ---- global -> registers -> LDS (rows past the operand read as zero) ----------------------
  // A: 16 blocks of 8 rows x 128 B, two per wave.  B unpacked: 32 such blocks, four per wave.
  // B packed: a wave load covers 16 rows x 64 B; two per wave; a lane's 16 bytes become the two
  // neighbouring 16-byte pieces 2p, 2p+1 of its row.
  constexpr int NLA = 2, NLB = PACKED ? 2 : 4;
  // two sets of staging registers: the loads of a stage are issued two stages ahead of its use and
  // written to LDS one stage ahead, so that a stage never waits for a load issued in it
  v4i sta[2][NLA], stb[2][NLB];
  auto row_swz = [](int row) { return (row ^ (row >> 3)) & 7; };
  auto load_stage = [&](const int set, int k0) {
#pragma unroll
    for (int i = 0; i < NLA; ++i) {
      const int row = (wave * NLA + i) * 8 + (lane >> 3);
      const int cb = (((lane & 7) ^ row_swz(row)) & 7) * 16;
      sta[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, row * (int)g.lda + cb, k0, 0);
    }
#pragma unroll
    for (int i = 0; i < NLB; ++i) {
      if constexpr (PACKED) {
        const int row = (wave * NLB + i) * 16 + (lane >> 2);
        stb[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, row * (int)g.ldb + (lane & 3) * 16, k0 / 2, 0);
      } else {
        const int row = (wave * NLB + i) * 8 + (lane >> 3);
        const int cb = (((lane & 7) ^ row_swz(row)) & 7) * 16;
        stb[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, row * (int)g.ldb + cb, k0, 0);
      }
    }
  };
  auto store_stage = [&](const int set, uint8_t* st) {
#pragma unroll
    for (int i = 0; i < NLA; ++i)
      *reinterpret_cast<v4i*>(st + (wave * NLA + i) * 1024 + lane * 16) = sta[set][i];
#pragma unroll
    for (int i = 0; i < NLB; ++i) {
      if constexpr (PACKED) {
        const int row = (wave * NLB + i) * 16 + (lane >> 2);
        const int p = lane & 3;
        // dword d of the load = k 8d..8d+7 of this lane's 32: even k in low nibbles.  Values * 16:
        // even k: (x << 4) & 0xF0F0F0F0, odd k: x & 0xF0F0F0F0; then bytes interleaved back to k order.
        v4i lo, hi;
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t x = (uint32_t)stb[set][i][d];
          const uint32_t ev = (x << 4) & 0xF0F0F0F0u, od = x & 0xF0F0F0F0u;
          const uint32_t k03 = __builtin_amdgcn_perm(od, ev, 0x05010400u);  // e0 o0 e1 o1
          const uint32_t k47 = __builtin_amdgcn_perm(od, ev, 0x07030602u);  // e2 o2 e3 o3
          if (d < 2) { lo[2 * d] = (int)k03; lo[2 * d + 1] = (int)k47; }
          else { hi[2 * (d - 2)] = (int)k03; hi[2 * (d - 2) + 1] = (int)k47; }
        }
        uint8_t* rowp = st + kATile + row * BK;
        *reinterpret_cast<v4i*>(rowp + (((2 * p) ^ row_swz(row)) * 16)) = lo;
        *reinterpret_cast<v4i*>(rowp + (((2 * p + 1) ^ row_swz(row)) * 16)) = hi;
      } else {
        *reinterpret_cast<v4i*>(st + kATile + (wave * NLB + i) * 1024 + lane * 16) = stb[set][i];
      }
    }
  };
  // group scales of the tile: thread t < 128 a row scale, 128 <= t < 384 a column scale
  float sc_reg = 1.0f;
  auto load_scales = [&](int grp) {
    sc_reg = 1.0f;
    if (grp < g.groups) {
      if (tid < GM) {
        if (m0 + tid < g.m) sc_reg = g.row_scale[(int64_t)grp * g.m + m0 + tid];
      } else if (tid < GM + GN) {
        const int64_t nn = n0 + (tid - GM);
        if (nn < g.n) sc_reg = g.col_scale[(int64_t)grp * g.n + nn] * (PACKED ? 0.0625f : 1.0f);
      }
    }
  };
  auto store_scales = [&](int buf) {
    if (tid < GM) srow[buf][tid] = sc_reg;
    else if (tid < GM + GN) scol[buf][tid - GM] = sc_reg;
  };

  // ---- fragments ---------------------------------------------------------------------------
  const int lf0 = (lr ^ (lr >> 3)) & 7;
  int frag_off[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) frag_off[c] = lr * BK + ((lh ^ lf0 ^ c) * 16);
  const int a_base = wm * 64 * BK, b_base = kATile + wn * 64 * BK;

  v16i acc[2][2];
  float sum[2][2][16];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc[mi][ni][r] = 0; sum[mi][ni][r] = 0.0f; }
  const v16i kZero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  const int nstages = g.groups * g.stages_per_group;
  load_stage(0, 0);
  load_scales(0);
  store_stage(0, stage_mem[0]);
  store_scales(0);
  if (nstages > 1) load_stage(1, BK);  // set 1 holds stage 1, set 0 will take stage 2, ...
  __syncthreads();
  // one stage; `set` holds the registers of stage s + 1, the other set takes the loads of s + 2
  auto stage = [&](const int s, const int set) {
    const int grp = ONE ? s : s / g.stages_per_group;
    const bool last_of_group = ONE || (s + 1) % g.stages_per_group == 0;
    const uint8_t* st = stage_mem[s & 1];
    if (s + 2 < nstages) load_stage(set ^ 1, (s + 2) * BK);
    if (last_of_group) load_scales(grp + 1);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      v4i fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int c = (2 * ks) ^ (4 * (i & 1));
        fa[i] = *reinterpret_cast<const v4i*>(st + a_base + i * 32 * BK + frag_off[c]);
        fb[i] = *reinterpret_cast<const v4i*>(st + b_base + i * 32 * BK + frag_off[c]);
      }
      // the first MFMA of a group starts from a zero accumulator operand instead of zeroed registers
      const bool fresh = ks == 0 && (ONE || (s % g.stages_per_group) == 0);
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
          if (fresh) acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], kZero, 0, 0, 0);
          else acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
        }
    }
    if (last_of_group) {
      // lane holds C[m = mi*32 + lr][n = ni*32 + 8q + 4lh + e], register 4q + e
      const int buf = grp & 1;
      float rs[2];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) rs[mi] = srow[buf][wm * 64 + mi * 32 + lr];
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const float4 cs4 = *reinterpret_cast<const float4*>(&scol[buf][wn * 64 + ni * 32 + 8 * q + 4 * lh]);
          const float cs[4] = {cs4.x, cs4.y, cs4.z, cs4.w};
#pragma unroll
          for (int mi = 0; mi < 2; ++mi)
#pragma unroll
            for (int e = 0; e < 4; e += 2) {
              // every product and the sum round on their own (the library is built with
              // floating-point contraction off, so no fused multiply-add appears here); values
              // are rounded two at a time (one packed conversion per pair)
              float f0 = (float)acc[mi][ni][4 * q + e], f1 = (float)acc[mi][ni][4 * q + e + 1];
              round_pair<kOutBf16>(f0, f1);
              f0 *= rs[mi]; f1 *= rs[mi];
              round_pair<kP1Bf16>(f0, f1);
              f0 *= cs[e]; f1 *= cs[e + 1];
              round_pair<kP2Bf16>(f0, f1);
              if constexpr (kOutBf16 && !kP2Bf16) round_pair<true>(f0, f1);  // final cast of the tile
              sum[mi][ni][4 * q + e] += f0;
              sum[mi][ni][4 * q + e + 1] += f1;
            }
        }
    }
    // the registers of stage s + 1 (requested a whole stage ago) go to the buffer stage s - 1 left;
    // the barrier is a bare s_barrier: a __syncthreads() would also wait for the loads of s + 2
    if (s + 1 < nstages) store_stage(set, stage_mem[(s + 1) & 1]);
    if (last_of_group) store_scales((grp + 1) & 1);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  for (int s = 0; s < nstages; s += 2) {
    stage(s, 1);
    if (s + 1 < nstages) stage(s + 1, 0);
  }

  // ---- output --------------------------------------------------------------------------------
  constexpr int kEsz = kOutBf16 ? 2 : 4;
  uint8_t* cb = reinterpret_cast<uint8_t*>(g.c);
  const bool vec = (g.ldc % 4) == 0 && ((uintptr_t)cb % 16) == 0;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
    const int64_t mm = m0 + wm * 64 + mi * 32 + lr;
    if (mm >= g.m) continue;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t nn = n0 + wn * 64 + ni * 32 + 8 * q + 4 * lh;
        if (nn >= g.n) continue;
        float o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = round_to<kOutBf16>(sum[mi][ni][4 * q + e]);
        uint8_t* dst = cb + (mm * g.ldc + nn) * kEsz;
        if (vec && nn + 4 <= g.n) {
          if constexpr (kOutBf16) {
            uint2 w;
            w.x = (uint32_t)bf16_bits(o[0]) | ((uint32_t)bf16_bits(o[1]) << 16);
            w.y = (uint32_t)bf16_bits(o[2]) | ((uint32_t)bf16_bits(o[3]) << 16);
            *reinterpret_cast<uint2*>(dst) = w;
          } else {
            *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
          }
        } else {
          for (int e = 0; e < 4 && nn + e < g.n; ++e) {
            if constexpr (kOutBf16) reinterpret_cast<uint16_t*>(dst)[e] = bf16_bits(o[e]);
            else reinterpret_cast<float*>(dst)[e] = o[e];
          }
        }
      }
  }
}

// [n][k] int4 values in int8 bytes -> [n][k/2] packed, low nibble = even k.
__global__ void pack_i4_kernel(const int8_t* src, uint8_t* dst, int64_t count2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count2) return;
  const uint32_t lo = (uint32_t)src[2 * i] & 0xFu, hi = (uint32_t)src[2 * i + 1] & 0xFu;
  dst[i] = (uint8_t)(lo | (hi << 4));
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_pack_i4(const void* src, void* dst, int64_t count, void* stream) {
  clear_error();
  AQTX_REQUIRE(count >= 0 && count % 2 == 0, "aqtx_pack_i4: count must be even and non-negative");
  if (count == 0) return 0;
  AQTX_REQUIRE(src != nullptr && dst != nullptr, "aqtx_pack_i4: NULL buffer");
  const int64_t n2 = count / 2;
  pack_i4_kernel<<<(unsigned)((n2 + 255) / 256), 256, 0, reinterpret_cast<hipStream_t>(stream)>>>(
      reinterpret_cast<const int8_t*>(src), reinterpret_cast<uint8_t*>(dst), n2);
  AQTX_HIP_CHECK_LAUNCH("pack_i4_kernel");
  return 0;
}

extern "C" int aqtx_gemm_i8_grouped(const aqtx_grouped_gemm_plan* p, const void* a, const void* b,
                                    const float* row_scale, const float* col_scale, void* c, void* stream) {
  clear_error();
  AQTX_REQUIRE(p != nullptr, "aqtx_gemm_i8_grouped: plan is NULL");
  AQTX_REQUIRE(p->m >= 0 && p->n >= 0 && p->k >= 0 && p->group > 0, "aqtx_gemm_i8_grouped: bad shape");
  AQTX_REQUIRE(p->a_dtype == AQTX_I8 || p->a_dtype == AQTX_I4, "aqtx_gemm_i8_grouped: a must be an int8 container");
  AQTX_REQUIRE(p->b_dtype == AQTX_I8 || p->b_dtype == AQTX_I4 || p->b_dtype == AQTX_I4P,
               "aqtx_gemm_i8_grouped: b must be int8, int4-in-int8 or packed int4");
  AQTX_REQUIRE(p->group % 128 == 0 && p->k % p->group == 0,
               "aqtx_gemm_i8_grouped: group (%lld) must be a multiple of 128 that divides k (%lld)",
               (long long)p->group, (long long)p->k);
  AQTX_REQUIRE(is_float_dtype(p->out_dtype) && is_float_dtype(p->row_scale_dtype) &&
                   is_float_dtype(p->col_scale_dtype),
               "aqtx_gemm_i8_grouped: out and scale dtypes must be bf16 or f32");
  const bool packed = p->b_dtype == AQTX_I4P;
  AQTX_REQUIRE(p->lda >= p->k && p->ldb >= (packed ? p->k / 2 : p->k) && p->ldc >= p->n,
               "aqtx_gemm_i8_grouped: leading dimension smaller than the row length");
  if (p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(a != nullptr && b != nullptr && c != nullptr && row_scale != nullptr && col_scale != nullptr,
               "aqtx_gemm_i8_grouped: NULL buffer");
  AQTX_REQUIRE(p->k > 0, "aqtx_gemm_i8_grouped: empty contraction");
  AQTX_REQUIRE((p->lda % 16 == 0) && (p->ldb % 16 == 0) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0),
               "aqtx_gemm_i8_grouped: operands must be 16-byte aligned with leading dimensions multiple of 16");
  AQTX_REQUIRE(p->lda * (int64_t)GM < (1ll << 31) && p->ldb * (int64_t)GN < (1ll << 31),
               "aqtx_gemm_i8_grouped: leading dimension too large for 32-bit tile offsets");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)c % esz) == 0, "aqtx_gemm_i8_grouped: output is not element aligned");

  GroupedArgs g{};
  g.a = reinterpret_cast<const uint8_t*>(a);
  g.b = reinterpret_cast<const uint8_t*>(b);
  g.row_scale = row_scale; g.col_scale = col_scale; g.c = c;
  g.m = p->m; g.n = p->n; g.k = p->k; g.lda = p->lda; g.ldb = p->ldb; g.ldc = p->ldc;
  g.groups = (int)(p->k / p->group);
  g.stages_per_group = (int)(p->group / 128);
  g.tiles_m = (int)((p->m + GM - 1) / GM);
  g.tiles_n = (int)((p->n + GN - 1) / GN);
  int epi;
  if (p->out_dtype == AQTX_F32) epi = 2;
  else if (p->row_scale_dtype != AQTX_BF16) epi = 1;
  else epi = p->col_scale_dtype == AQTX_BF16 ? 0 : 4;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n));
  // the compile-time form of the one-stage group costs the unpacked variant a few spilled registers
  const bool one = g.stages_per_group == 1 && packed;
#define AQTX_LAUNCH(E)                                                       \
  do {                                                                      \
    if (packed && one) gemm_grouped_kernel<E, true, true><<<grid, 512, 0, st>>>(g);         \
    else if (packed) gemm_grouped_kernel<E, true, false><<<grid, 512, 0, st>>>(g);          \
    else if (one) gemm_grouped_kernel<E, false, true><<<grid, 512, 0, st>>>(g);             \
    else gemm_grouped_kernel<E, false, false><<<grid, 512, 0, st>>>(g);                     \
  } while (0)
  switch (epi) {
    case 0: AQTX_LAUNCH(0); break;
    case 1: AQTX_LAUNCH(1); break;
    case 2: AQTX_LAUNCH(2); break;
    default: AQTX_LAUNCH(4); break;
  }
#undef AQTX_LAUNCH
  AQTX_HIP_CHECK_LAUNCH("gemm_grouped_kernel");
  return 0;
}

// int8 x int8 -> int32 contraction for shapes with few output tiles: the same arithmetic as the
// 256 x 256 kernel of gemm_core.h on 128 x 128 tiles, optionally with K cut into slices.
//
// A 256 x 256 tile keeps one CU busy for all of K whatever the rest of the chip does, so a product
// of 512 x 4096 (32 such tiles) leaves 224 of the 256 CUs idle.  Here a workgroup of 8 waves (4 x 2)
// owns 128 x 128 of C, a wave 32 x 64 (two v_mfma_i32_32x32x32_i8 tiles, 32 accumulators), with 128
// registers per lane and 72 KiB of LDS, so that two workgroups share a CU: four times the workgroups,
// each a quarter of the work.  When even that leaves CUs idle and K is long, grid.z cuts K into slices
// whose int32 partial sums go to slabs of a workspace, and dequant_slabs_kernel adds them up (integer
// sums: exact in any order) and applies the epilogue.
//
// LDS rows are 144 bytes apart (128 of data, 16 of padding): the 16 lanes of a fragment read fall into
// distinct banks and every address of the loop is a loop-invariant register plus an immediate.
#include "gemm_core.h"

namespace aqtx {
namespace {

constexpr int TM = 128, TN = 128;
constexpr int kRow = BK + 16;
constexpr int kATile = TM * kRow, kBTile = TN * kRow, kStage = kATile + kBTile;  // 36 KiB

// MMA, EPI, COL_FIRST as in gemm_kernel.  PACKED: a row of B has half the bytes in memory that it has in LDS:
// int4 values two per byte (see gemm_kernel's BPACK), or, with MmaBf16W8, int8 values that become bf16 (A then
// holds bf16 values, and GemmArgs::k, lda and stride_a count its bytes), or, with MmaBf16F8, fp8 bytes that become
// bf16; A's rows are then widened the same way (MMA::kWidenA: GemmArgs::k counts the bf16 bytes of a row in LDS,
// twice the fp8 bytes in memory, while lda and stride_a count those).
// SLAB: this launch writes raw partial sums of a K slice to its slab (EPI is 3 then; integer sums only).
// CONV: A is a convolution input read in place (GemmArgs::conv): the window gather that would otherwise be
// materialised (features % 128 == 0, so a 128-byte stage lies inside one tap).
template <class MMA, int EPI, bool COL_FIRST, bool PACKED, bool SLAB, bool CONV = false>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
void gemm_mid_kernel(const GemmArgs g_in) {
  static_assert(!SLAB || EPI == 3, "a K slice leaves raw sums");
  static_assert(!CONV || (MMA::kIntAcc && !PACKED && !SLAB), "the convolution reads int8 bytes, whole K");
  static_assert(MMA::kIntAcc || (!SLAB && PACKED == MMA::kWidenB && EPI != 3), "float sums: whole K; fp8 bytes as they are");
  constexpr bool WIDEN_A = MMA::kWidenA;
  static_assert(!WIDEN_A || (PACKED && !CONV), "a widened A goes with a widened B");
  using Acc = typename MMA::Acc;
  using AccScalar = typename MMA::AccScalar;
  using Frag = typename MMA::Frag;
  constexpr int kChunks = MMA::kChunks;  // 16-byte chunks a lane holds of one MFMA's k
  GemmArgs g = g_in;
  __shared__ __attribute__((aligned(1024))) uint8_t stage_mem[2 * kStage];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;  // 32 rows, 64 columns
  const int lr = lane & 31, lh = lane >> 5;
  int tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t bz = blockIdx.y;
  const int64_t m0 = (int64_t)tm * TM, n0 = (int64_t)tn * TN;
  if constexpr (SLAB) {  // this workgroup's slice of K
    const int64_t kb = (int64_t)blockIdx.z * g.k_chunk;
    g.a += kb;
    g.b += g.b_frag ? (PACKED ? kb / 2 : kb) * 16 : (PACKED ? kb / 2 : kb);  // 64 bytes of a row = one KiB step
    g.k = (g.k - kb) < g.k_chunk ? (g.k - kb) : g.k_chunk;
  }
  const int64_t rows_a = (g.m - m0) < TM ? (g.m - m0) : TM;
  const int64_t rows_b = (g.n - n0) < TN ? (g.n - n0) : TN;
  const int kb_bytes = PACKED ? (int)(g.k / 2) : (int)g.k;  // bytes of one B row (of this slice)
  const __amdgpu_buffer_rsrc_t rsrc_a = CONV
      ? __builtin_amdgcn_make_buffer_rsrc((void*)g.a, 0, (int)g.conv.x_bytes, kBufferRsrcWord3)
      : __builtin_amdgcn_make_buffer_rsrc((void*)(g.a + bz * g.stride_a + m0 * g.lda), 0,
                                          (int)((rows_a - 1) * g.lda + (WIDEN_A ? g.k / 2 : g.k)), kBufferRsrcWord3);
  const int64_t blocks_b = (rows_b + 15) / 16;  // fragment order: the tile's 16-row blocks, whole
  const __amdgpu_buffer_rsrc_t rsrc_b = g.b_frag
      ? __builtin_amdgcn_make_buffer_rsrc((void*)(g.b + (n0 / 16) * (int64_t)g.b_steps * 1024), 0,
                                          (int)(blocks_b * g.b_steps * 1024), kBufferRsrcWord3)
      : __builtin_amdgcn_make_buffer_rsrc((void*)(g.b + bz * g.stride_b + n0 * g.ldb), 0,
                                          (int)((rows_b - 1) * g.ldb + kb_bytes), kBufferRsrcWord3);

  // ---- global -> registers -> LDS (rows past the operand read as zero, and so do the 16-byte chunks
  // past K in the last stage).  A: 16 blocks of 8 rows x 128 B, two per wave.  B unpacked: the same.
  // B packed: a wave load covers 16 rows x 64 B, one per wave; a lane's 16 bytes become the 32 bytes at
  // 32 * (lane & 3) of its row.  The row and chunk of a load are in its vector offset, which the buffer's
  // range check covers; the scalar offset (the stage's k) is not range checked, the mask on K covers it.
  constexpr int NLA = WIDEN_A ? 1 : 2, NLB = PACKED ? 1 : 2, NL = NLA + NLB;
  constexpr int kOutside = 0x7FFFFFF0;
  v4i stg[NL];
  const int ld_a = WIDEN_A ? (wave * 16 + (lane >> 2)) * (int)g.lda + (lane & 3) * 16
                           : (wave * 16 + (lane >> 3)) * (int)g.lda + (lane & 7) * 16;
  // B in fragment order: a wave load is one KiB = 64 bytes of 16 rows (lane -> row lane & 15, bytes 16 (lane >> 4));
  // unpacked, the wave's two loads are the two KiB of a stage (the second 64 bytes further in LDS), and the
  // scalar offset advances one KiB per 64 row bytes
  const int ld_b = g.b_frag ? wave * g.b_steps * 1024 + lane * 16
                 : PACKED ? (wave * 16 + (lane >> 2)) * (int)g.ldb + (lane & 3) * 16
                          : (wave * 16 + (lane >> 3)) * (int)g.ldb + (lane & 7) * 16;
  const int ld_b_next = g.b_frag ? 1024 : 8 * (int)g.ldb;  // the wave's second load (unpacked)
  const int kpos_a = WIDEN_A ? (lane & 3) * 32 : (lane & 7) * 16;
  const int kpos_b = g.b_frag ? (lane >> 4) * (PACKED ? 32 : 16) : PACKED ? (lane & 3) * 32 : (lane & 7) * 16;
  const int kpos_b_next = g.b_frag ? 64 : 0;
  const int st_a = WIDEN_A ? (wave * 16 + (lane >> 2)) * kRow + (lane & 3) * 32
                           : (wave * 16 + (lane >> 3)) * kRow + (lane & 7) * 16;
  const int st_b = kATile + (g.b_frag ? (wave * 16 + (lane & 15)) * kRow + (lane >> 4) * (PACKED ? 32 : 16)
                             : PACKED ? (wave * 16 + (lane >> 2)) * kRow + (lane & 3) * 32
                                      : (wave * 16 + (lane >> 3)) * kRow + (lane & 7) * 16);
  const int st_b_next = g.b_frag ? 64 : 8 * kRow;
  const int ksh_b = g.b_frag ? 4 : 0;  // scalar offset of B = row bytes << ksh_b
  // CONV: position of this lane's two rows (first corner of their windows, in input coordinates) and the tap
  // the next request belongs to, advanced one stage per request (requests come in stage order)
  int cpix[2] = {0, 0}, ci0[2] = {0, 0}, ci1[2] = {0, 0}, ci2[2] = {0, 0};
  int ct0 = 0, ct1 = 0, ct2 = 0, cch = 0;  // wave-uniform
  if constexpr (CONV) {
#pragma unroll
    for (int j = 0; j < NLA; ++j) {
      int64_t row = m0 + wave * 16 + (lane >> 3) + j * 8;
      const bool in = row < g.m;
      if (!in) row = 0;
      const int o2 = (int)(row % g.conv.osz[2]); row /= g.conv.osz[2];
      const int o1 = (int)(row % g.conv.osz[1]); row /= g.conv.osz[1];
      const int o0 = (int)(row % g.conv.osz[0]); row /= g.conv.osz[0];
      ci0[j] = in ? o0 * g.conv.str[0] - g.conv.pad[0] : -(1 << 28);  // rows past m: outside for every tap
      ci1[j] = o1 * g.conv.str[1] - g.conv.pad[1];
      ci2[j] = o2 * g.conv.str[2] - g.conv.pad[2];
      cpix[j] = in ? (int)((((row * g.conv.in[0] + ci0[j]) * g.conv.in[1] + ci1[j]) * g.conv.in[2] + ci2[j]) * g.conv.c) : 0;
    }
  }
  auto conv_advance = [&]() {
    cch += BK;
    if (cch >= g.conv.c) {
      cch = 0;
      if (++ct2 == g.conv.ker[2]) { ct2 = 0; if (++ct1 == g.conv.ker[1]) { ct1 = 0; ++ct0; } }
    }
  };
  auto load_one = [&](const int j, int k0) {
    if constexpr (CONV) {
      if (j < NLA) {
        const int d0 = ct0 * g.conv.dil[0], d1 = ct1 * g.conv.dil[1], d2 = ct2 * g.conv.dil[2];
        const bool in = (unsigned)(ci0[j] + d0) < (unsigned)g.conv.in[0] && (unsigned)(ci1[j] + d1) < (unsigned)g.conv.in[1] &&
                        (unsigned)(ci2[j] + d2) < (unsigned)g.conv.in[2] && ct0 < g.conv.ker[0];
        const int tap = ((d0 * g.conv.in[1] + d1) * g.conv.in[2] + d2) * g.conv.c + cch;
        stg[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, in ? cpix[j] + tap + kpos_a : kOutside, 0, 0);
        return;
      }
    }
    if (j < NLA) {
      const int vo = k0 + kpos_a < (int)g.k ? ld_a + j * 8 * (int)g.lda : kOutside;
      stg[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, vo, WIDEN_A ? k0 / 2 : k0, 0);
    } else if constexpr (PACKED) {
      const int vo = k0 + kpos_b < (int)g.k ? ld_b : kOutside;
      stg[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, (k0 / 2) << ksh_b, 0);
    } else {
      const int vo = k0 + kpos_b + (j - NLA) * kpos_b_next < (int)g.k ? ld_b + (j - NLA) * ld_b_next : kOutside;
      stg[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, k0 << ksh_b, 0);
    }
  };
  auto store_stage = [&](const int stage_base) {
    uint8_t* st = stage_mem + stage_base;
    if constexpr (WIDEN_A) {
      v4i lo, hi;
      MMA::widen_a(stg[0], lo, hi);
      *reinterpret_cast<v4i*>(st + st_a) = lo;
      *reinterpret_cast<v4i*>(st + st_a + 16) = hi;
    } else {
#pragma unroll
      for (int j = 0; j < NLA; ++j) *reinterpret_cast<v4i*>(st + st_a + j * 8 * kRow) = stg[j];
    }
    if constexpr (PACKED) {
      v4i lo, hi;
      if constexpr (MMA::kWidenB) MMA::widen_b(stg[NLA], lo, hi);
      else unpack_i4x32(stg[NLA], lo, hi, g.a_even_odd8);
      *reinterpret_cast<v4i*>(st + st_b) = lo;
      *reinterpret_cast<v4i*>(st + st_b + 16) = hi;
    } else {
#pragma unroll
      for (int j = 0; j < NLB; ++j) *reinterpret_cast<v4i*>(st + st_b + j * st_b_next) = stg[NLA + j];
    }
  };

  // fragment of k step ks: 16 kChunks bytes at (32 ks + 16 lh) kChunks of row lr of the 32-row block
  const int a_off = (wm * 32 + lr) * kRow + lh * 16 * kChunks;
  const int b_off = kATile + (wn * 64 + lr) * kRow + lh * 16 * kChunks;
  auto frag = [&](const uint8_t* at) -> Frag {
    if constexpr (kChunks == 1) {
      return *reinterpret_cast<const v4i*>(at);
    } else {
      const v4i x0 = *reinterpret_cast<const v4i*>(at), x1 = *reinterpret_cast<const v4i*>(at + 16);
      return Frag{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
  };

  Acc acc[2];
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc[0][r] = 0; acc[1][r] = 0; }

  const int nstages = (int)((g.k + BK - 1) / BK);
#pragma unroll
  for (int j = 0; j < NL; ++j) load_one(j, 0);
  if constexpr (CONV) conv_advance();
  store_stage(0);
#pragma unroll
  for (int j = 0; j < NL; ++j) load_one(j, nstages > 1 ? BK : 0);
  if constexpr (CONV) conv_advance();
  __syncthreads();

  // Stage s reads buffer BUF; the staging registers (stage s + 1, requested during stage s - 1) go to the
  // buffer stage s - 1 left, and the loads of stage s + 2 are issued behind them.  Past the last stage
  // the store and the loads are repeated harmlessly (a buffer nobody reads, k offset 0) rather than
  // branched around.
  auto stage = [&](const int s, auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    const uint8_t* st = stage_mem + BUF * kStage;
#pragma unroll
    for (int ks = 0; ks < 4 / kChunks; ++ks) {
      const Frag fa = frag(st + a_off + ks * 32 * kChunks);
      const Frag fb0 = frag(st + b_off + ks * 32 * kChunks);
      const Frag fb1 = frag(st + b_off + 32 * kRow + ks * 32 * kChunks);
      acc[0] = MMA::mma(fb0, fa, acc[0]);
      acc[1] = MMA::mma(fb1, fa, acc[1]);
    }
    store_stage((1 - BUF) * kStage);
    const int k_next = s + 2 < nstages ? (s + 2) * BK : 0;
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(j, k_next);
    if constexpr (CONV) conv_advance();  // past the last stage the tap leaves the window: zeros nobody reads
    // a bare s_barrier: a __syncthreads() would also wait for the global loads just issued
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  for (int s = 0; s < nstages; s += 2) {
    stage(s, std::integral_constant<int, 0>{});
    if (s + 1 < nstages) stage(s + 1, std::integral_constant<int, 1>{});
  }

  // ---- epilogue: lane holds C[m = wm*32 + lr][n = wn*64 + ni*32 + 8q + 4lh + e], register 4q + e of tile ni
  const int64_t mm = m0 + wm * 32 + lr;
  if (mm >= g.m) return;
  if constexpr (SLAB) {
    int32_t* dst = g.slabs + (((int64_t)blockIdx.z * gridDim.y + bz) * g.m + mm) * g.n;
    const bool vec = (g.n % 4) == 0;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t nn = n0 + wn * 64 + ni * 32 + 8 * q + 4 * lh;
        if (nn >= g.n) continue;
        int v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = PACKED ? acc[ni][4 * q + e] >> 4 : acc[ni][4 * q + e];  // exact: multiples of 16 (SLAB: int4)
        if (vec) *reinterpret_cast<int4*>(dst + nn) = make_int4(v[0], v[1], v[2], v[3]);
        else for (int e = 0; e < 4 && nn + e < g.n; ++e) dst[nn + e] = v[e];
      }
    return;
  } else {
    constexpr bool kOutBf16 = EPI <= 1 || EPI == 4;
    constexpr int kEsz = kOutBf16 ? 2 : 4;
    const int64_t row_o = bz * g.stride_c + mm * g.ldc;
    const float s_row = g.row_scale ? g.row_scale[bz * g.stride_rs + mm] : 1.0f;
    const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
    const bool cs_vec = ((uintptr_t)cs % 16) == 0;
    const bool acc_vec = (g.ldc % 4) == 0 && (g.stride_c % 4) == 0 && ((uintptr_t)g.acc_out % 16) == 0;
    const bool c_vec = (g.ldc % 4) == 0 && (g.stride_c % 4) == 0 && ((uintptr_t)g.c % (4 * kEsz)) == 0;
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int64_t nn = n0 + wn * 64 + ni * 32 + 8 * q + 4 * lh;
        if (nn >= g.n) continue;
        const bool full = nn + 4 <= g.n;
        AccScalar v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          if constexpr (PACKED && MMA::kIntAcc) v[e] = acc[ni][4 * q + e] >> 4;
          else v[e] = acc[ni][4 * q + e];
        }
        if (g.acc_out != nullptr) {  // 32-bit patterns, int32 or float
          AccScalar* dst = reinterpret_cast<AccScalar*>(g.acc_out) + row_o + nn;
          if (full && acc_vec) {
            *reinterpret_cast<int4*>(dst) = make_int4(__builtin_bit_cast(int, v[0]), __builtin_bit_cast(int, v[1]),
                                                      __builtin_bit_cast(int, v[2]), __builtin_bit_cast(int, v[3]));
          } else {
            for (int e = 0; e < 4 && nn + e < g.n; ++e) dst[e] = v[e];
          }
        }
        uint8_t* dst = reinterpret_cast<uint8_t*>(g.c) + (row_o + nn) * kEsz;
        if constexpr (EPI == 3) {
          if (full && c_vec) *reinterpret_cast<int4*>(dst) = make_int4(v[0], v[1], v[2], v[3]);
          else for (int e = 0; e < 4 && nn + e < g.n; ++e) reinterpret_cast<int32_t*>(dst)[e] = v[e];
        } else {
          float csv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
          if (cs != nullptr) {
            if (full && cs_vec) {
              const float4 c4 = *reinterpret_cast<const float4*>(cs + nn);
              csv[0] = c4.x; csv[1] = c4.y; csv[2] = c4.z; csv[3] = c4.w;
            } else {
              for (int e = 0; e < 4 && nn + e < g.n; ++e) csv[e] = cs[nn + e];
            }
          }
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) o[e] = dequant_value<EPI, COL_FIRST>(v[e], s_row, csv[e]);
          if (full && c_vec) {
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
}

template <int EPI, bool COL_FIRST>
void launch_mid(const GemmArgs& g, bool packed, dim3 grid, hipStream_t st) {
  if constexpr (!COL_FIRST) {
    if (packed) { gemm_mid_kernel<MmaI8, EPI, false, true, false><<<grid, 512, 0, st>>>(g); return; }
  }
  gemm_mid_kernel<MmaI8, EPI, COL_FIRST, false, false><<<grid, 512, 0, st>>>(g);
}

template <class MMA, bool WIDENED = false>
void launch_mid_fp8(const GemmArgs& g, int epi, dim3 grid, hipStream_t st) {
#define AQTX_MID8(E) do { if (g.col_first) gemm_mid_kernel<MMA, E, true, WIDENED, false><<<grid, 512, 0, st>>>(g); \
                          else gemm_mid_kernel<MMA, E, false, WIDENED, false><<<grid, 512, 0, st>>>(g); } while (0)
  switch (epi) {
    case 0: AQTX_MID8(0); break;
    case 1: AQTX_MID8(1); break;
    case 4: AQTX_MID8(4); break;
    default: AQTX_MID8(2); break;
  }
#undef AQTX_MID8
}

template <int EPI>
void launch_slab_sum(const GemmArgs& g, dim3 grid, hipStream_t st) {
  if constexpr (EPI != 3) {
    if (g.col_first) { dequant_slabs_kernel<EPI, true><<<grid, 256, 0, st>>>(g); return; }
  }
  dequant_slabs_kernel<EPI, false><<<grid, 256, 0, st>>>(g);
}

}  // namespace

// Whether the 128 x 128 kernel takes the plan (0 = no) and in how many slices of K (1 = none).
int gemm_mid_k_slices(const aqtx_gemm_plan* p) {
  if (p->group_offsets != nullptr || (p->tuning != 0 && p->tuning != 128) || !gemm_vector_shape_ok(p)) return 0;  // 4, 8, 16: the large tiles
  if (p->b_dtype == AQTX_I4P && p->scale_order != AQTX_SCALE_ROW_THEN_COL) return 0;
  if (p->lda * (int64_t)TM >= (1ll << 31) || p->ldb * (int64_t)TN >= (1ll << 31)) return 0;
  const int64_t pad256 = ((p->m + BM - 1) / BM) * ((p->n + BN - 1) / BN);
  const int64_t pad128 = ((p->m + TM - 1) / TM) * ((p->n + TN - 1) / TN);
  const int64_t tiles256 = pad256 * p->batch, tiles128 = pad128 * p->batch;
  const int64_t max_by_k = (p->k + 2 * BK - 1) / (2 * BK);  // a slice holds at least two stages
  if (p->k_split > 1) return (int)(p->k_split < max_by_k ? p->k_split : max_by_k);
  // the large tiles fill the chip, unless a third of their area or more lies outside C (n or m of 128, say)
  const bool padded = 4 * pad256 * 2 >= 3 * pad128;
  if (p->tuning != 128 && tiles256 > 128 && !padded) return 0;
  if (p->k_split == 1 || tiles256 > 128) return 1;
  // slices until about 256 workgroups exist (one per CU; two fit), each walking at least 1024 of k; the
  // slabs they write and the sum kernel reads stay small next to the operands at such tile counts
  int64_t s = 256 / tiles128;
  if (s > 8) s = 8;
  if (s > p->k / 1024) s = p->k / 1024;
  return s < 1 ? 1 : (int)s;
}

int launch_gemm_i8_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                       const float* col_scale, void* c, int32_t* acc_out, int slices, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  g.a_even_odd8 = p->a_k_order == AQTX_K_EVEN_ODD8;
  g.tiles_m = (int)((p->m + TM - 1) / TM);
  g.tiles_n = (int)((p->n + TN - 1) / TN);
  const bool packed = p->b_dtype == AQTX_I4P;
  g.b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  g.b_steps = (int)(((packed ? p->k / 2 : p->k) + 63) / 64);
  const int epi = gemm_epilogue_id(p);
  if (epi < 0)
    return set_error("aqtx_gemm_i8: unsupported out/dequant/scale dtype combination (%d, %d, %d)",
                     p->out_dtype, p->dequant_dtype, p->row_scale_dtype);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  if (slices > 1) {
    const int64_t need = (int64_t)slices * p->batch * p->m * p->n * 4;
    AQTX_REQUIRE(p->k_split_workspace != nullptr && p->k_split_workspace_bytes >= need &&
                     ((uintptr_t)p->k_split_workspace % 16) == 0,
                 "aqtx_gemm_i8: %d slices of k need a 16-byte aligned k_split_workspace of %lld bytes", slices,
                 (long long)need);
    AQTX_REQUIRE(p->m <= 65535, "aqtx_gemm_i8: slices of k take at most 65535 rows (m = %lld); set k_split = 1",
                 (long long)p->m);
    g.k_split = slices;
    g.k_chunk = ((p->k + slices - 1) / slices + BK - 1) / BK * BK;
    g.k_split = (int)((p->k + g.k_chunk - 1) / g.k_chunk);
    g.slabs = reinterpret_cast<int32_t*>(p->k_split_workspace);
    grid.z = (unsigned)g.k_split;
    if (packed) gemm_mid_kernel<MmaI8, 3, false, true, true><<<grid, 512, 0, st>>>(g);
    else gemm_mid_kernel<MmaI8, 3, false, false, true><<<grid, 512, 0, st>>>(g);
    const dim3 egrid((unsigned)((p->n + 1023) / 1024), (unsigned)p->m, (unsigned)p->batch);
    switch (epi) {
      case 0: launch_slab_sum<0>(g, egrid, st); break;
      case 1: launch_slab_sum<1>(g, egrid, st); break;
      case 2: launch_slab_sum<2>(g, egrid, st); break;
      case 4: launch_slab_sum<4>(g, egrid, st); break;
      default: launch_slab_sum<3>(g, egrid, st); break;
    }
    AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel, k slices");
    return 0;
  }
  switch (epi) {
    case 0: if (g.col_first) launch_mid<0, true>(g, packed, grid, st); else launch_mid<0, false>(g, packed, grid, st); break;
    case 1: if (g.col_first) launch_mid<1, true>(g, packed, grid, st); else launch_mid<1, false>(g, packed, grid, st); break;
    case 2: if (g.col_first) launch_mid<2, true>(g, packed, grid, st); else launch_mid<2, false>(g, packed, grid, st); break;
    case 4: if (g.col_first) launch_mid<4, true>(g, packed, grid, st); else launch_mid<4, false>(g, packed, grid, st); break;
    default: launch_mid<3, false>(g, packed, grid, st); break;
  }
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel");
  return 0;
}

// Convolution of int8 operands without the window matrix: `w` describes the windows, `p` the contraction
// they amount to (m = images * positions, n = output features, k = taps * features).
int launch_conv_i8_mid(const aqtx_im2col_plan* w, const aqtx_gemm_plan* p, const void* x, const void* b,
                       const float* row_scale, const float* col_scale, void* c, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, x, b, row_scale, col_scale, c, nullptr);
  g.tiles_m = (int)((p->m + TM - 1) / TM);
  g.tiles_n = (int)((p->n + TN - 1) / TN);
  g.conv.c = w->c;
  int64_t in_elems = 1;
  for (int d = 0; d < 3; ++d) {
    const int s = d - (3 - w->rank);  // missing leading axes have extent 1
    g.conv.in[d] = s < 0 ? 1 : w->in_size[s];
    g.conv.ker[d] = s < 0 ? 1 : w->kernel[s];
    g.conv.str[d] = s < 0 ? 1 : w->stride[s];
    g.conv.dil[d] = s < 0 ? 1 : w->dilation[s];
    g.conv.pad[d] = s < 0 ? 0 : w->pad_lo[s];
    g.conv.osz[d] = s < 0 ? 1 : w->out_size[s];
    in_elems *= g.conv.in[d];
  }
  g.conv.x_bytes = w->n * in_elems * w->c;
  const int epi = gemm_epilogue_id(p);
  if (epi < 0 || epi == 3)
    return set_error("aqtx_conv_i8: unsupported out/dequant/scale dtype combination (%d, %d, %d)", p->out_dtype,
                     p->dequant_dtype, p->row_scale_dtype);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), 1);
#define AQTX_CONV(E) do { if (g.col_first) gemm_mid_kernel<MmaI8, E, true, false, false, true><<<grid, 512, 0, st>>>(g); \
                          else gemm_mid_kernel<MmaI8, E, false, false, false, true><<<grid, 512, 0, st>>>(g); } while (0)
  switch (epi) {
    case 0: AQTX_CONV(0); break;
    case 1: AQTX_CONV(1); break;
    case 4: AQTX_CONV(4); break;
    default: AQTX_CONV(2); break;
  }
#undef AQTX_CONV
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel<conv>");
  return 0;
}

// fp8 operands on the 128 x 128 tiles (float sums: K is never cut).
int launch_gemm_fp8_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                        const float* col_scale, void* c, float* acc_out, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  g.tiles_m = (int)((p->m + TM - 1) / TM);
  g.tiles_n = (int)((p->n + TN - 1) / TN);
  const int epi = gemm_epilogue_id(p);
  if (epi < 0 || epi == 3)
    return set_error("aqtx_gemm_fp8: unsupported out/dequant/scale dtype combination (%d, %d, %d)",
                     p->out_dtype, p->dequant_dtype, p->row_scale_dtype);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  const bool a5 = p->a_dtype == AQTX_E5M2, b5 = p->b_dtype == AQTX_E5M2;
  if (!a5 && !b5) launch_mid_fp8<MmaF8<0, 0>>(g, epi, grid, st);
  else if (!a5 && b5) launch_mid_fp8<MmaF8<0, 1>>(g, epi, grid, st);
  else if (a5 && !b5) launch_mid_fp8<MmaF8<1, 0>>(g, epi, grid, st);
  else launch_mid_fp8<MmaF8<1, 1>>(g, epi, grid, st);
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel<fp8>");
  return 0;
}

// fp8 operands contracted through bf16 (both widened in registers, float32-like sums) on the 128 x 128 tiles,
// whatever the number of tiles.
int launch_gemm_fp8_f32sum_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                               const float* col_scale, void* c, float* acc_out, hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, row_scale, col_scale, c, acc_out);
  g.k *= 2;  // bf16 bytes of a row in LDS; lda, ldb and the batch strides stay in fp8 bytes
  g.tiles_m = (int)((p->m + TM - 1) / TM);
  g.tiles_n = (int)((p->n + TN - 1) / TN);
  const int epi = gemm_epilogue_id(p);
  if (epi < 0 || epi == 3)
    return set_error("aqtx_gemm_fp8: unsupported out/dequant/scale dtype combination (%d, %d, %d)",
                     p->out_dtype, p->dequant_dtype, p->row_scale_dtype);
  AQTX_REQUIRE(p->lda * (int64_t)TM < (1ll << 31) && p->ldb * (int64_t)TN < (1ll << 31) && p->k < (1ll << 29),
               "aqtx_gemm_fp8: leading dimension or k too large for 32-bit tile offsets");
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  const bool a5 = p->a_dtype == AQTX_E5M2, b5 = p->b_dtype == AQTX_E5M2;
  if (!a5 && !b5) launch_mid_fp8<MmaBf16F8<0, 0>, true>(g, epi, grid, st);
  else if (!a5 && b5) launch_mid_fp8<MmaBf16F8<0, 1>, true>(g, epi, grid, st);
  else if (a5 && !b5) launch_mid_fp8<MmaBf16F8<1, 0>, true>(g, epi, grid, st);
  else launch_mid_fp8<MmaBf16F8<1, 1>, true>(g, epi, grid, st);
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel<fp8 through bf16>");
  return 0;
}

// Weight-only contraction (bf16 A, int8 B widened in registers, float sums) on the 128 x 128 tiles.  The
// epilogue is QTensor.dequant with the rhs scale alone: the sum in bf16, times the column scale in the
// promoted dtype, cast to bf16 (a missing row scale multiplies by one and rounds nothing).
int launch_gemm_weight_only_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* col_scale, void* c,
                                hipStream_t st) {
  GemmArgs g = make_gemm_args(p, a, b, nullptr, col_scale, c, nullptr);
  g.k *= 2; g.lda *= 2; g.stride_a *= 2;  // A in bytes
  g.col_first = 0;
  g.b_frag = p->b_layout == AQTX_W_FRAGMENTS;
  g.b_steps = (int)((p->k + 63) / 64);
  g.tiles_m = (int)((p->m + TM - 1) / TM);
  g.tiles_n = (int)((p->n + TN - 1) / TN);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  if (p->col_scale_dtype == AQTX_BF16) gemm_mid_kernel<MmaBf16W8, 0, false, true, false><<<grid, 512, 0, st>>>(g);
  else gemm_mid_kernel<MmaBf16W8, 4, false, true, false><<<grid, 512, 0, st>>>(g);
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel<weight only>");
  return 0;
}

}  // namespace aqtx

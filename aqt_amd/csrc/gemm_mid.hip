// int8 x int8 -> int32 contraction for shapes with few output tiles: the same arithmetic as the
// 256 x 256 kernel of gemm_core.h on smaller tiles, optionally with K cut into slices.
//
// A 256 x 256 tile keeps one CU busy for all of K whatever the rest of the chip does, so a product
// of 512 x 4096 (32 such tiles) leaves 224 of the 256 CUs idle.  Here a workgroup owns a tile of 128 x 128
// (8 waves of 32 x 64: two v_mfma_i32_32x32x32_i8 tiles, 32 accumulators), 64 x 128 or 64 x 64 (4 waves) of C:
// MidShape.  Two schedules.  Plain: two LDS buffers (72 KiB) and under 128 registers, so that two workgroups
// share a CU and fill each other's waits; for launches with more tiles than CUs.  Ring: three or four LDS
// buffers refilled group by group over the stage (unpacked operands by buffer loads straight into LDS, packed
// ones through three stages' worth of staging registers), for launches of at most one workgroup per CU, which
// has nobody to overlap its waits with.  When even the small tiles leave
// CUs idle and K is long, grid.z cuts K into slices whose int32 partial sums go to slabs of a workspace, and
// dequant_slabs_kernel adds them up (integer sums: exact in any order) and applies the epilogue.
//
// LDS rows of the plain schedule are 144 bytes apart (128 of data, 16 of padding): the 16 lanes of a fragment
// read fall into distinct banks and every address of the loop is a loop-invariant register plus an immediate.
// The ring shapes keep 128-byte rows with their 16-byte chunks swizzled instead, so that 8 rows are 1 KiB of
// consecutive LDS, which is what a buffer load straight into LDS fills.
#include "gemm_core.h"

namespace aqtx {
namespace {

constexpr int TM = 128, TN = 128;

// Tile of a workgroup and how its waves share it: WM x WN waves, each (TM / WM) x (TN / WN) of C in 32 x 32
// matrix-instruction tiles.  A wave fetches TM / waves rows of A and TN / waves rows of B per stage.
template <int TM_, int TN_, int WM_, int WN_, int OCC_ = 4, bool RING_ = false, int GROUP_ = 1, bool SWIZZLE_ = false,
          int BUFFERS_ = 0, bool PAIR_ = false>
struct MidShape {
  // direct ring: one barrier for every two stages (see the kernel)
  static constexpr bool kPair = PAIR_;
  // > 0 (ring, swizzled rows): operands that need no unpacking are requested straight into this many LDS
  // buffers (see the kernel); packed operands keep three buffers and the staging registers
  static constexpr int kBuffers = BUFFERS_;
  // LDS rows: 128 bytes of data and 16 of padding, or (kSwizzle) 128 bytes with the 16-byte chunks of a row
  // exchanged among themselves by an XOR with a function of the row, which spreads the 16 rows of a fragment
  // read over the banks just as well and fits three buffers of a 128 x 256 tile into the 160 KiB of a CU
  static constexpr bool kSwizzle = SWIZZLE_;
  static constexpr int kRow = SWIZZLE_ ? BK : BK + 16;
  static constexpr int kOcc = OCC_;      // waves per SIMD the registers are budgeted for
  static constexpr bool kRing = RING_;   // three LDS buffers and three stages in flight in registers (see the kernel)
  static constexpr int kGroup = GROUP_;  // ring schedule: k steps whose fragments are read together
  static constexpr int kTM = TM_, kTN = TN_, kWM = WM_, kWN = WN_, kWaves = WM_ * WN_, kThreads = 64 * kWaves;
  static constexpr int kIM = TM_ / WM_ / 32, kIN = TN_ / WN_ / 32;  // 32 x 32 tiles of a wave
  static constexpr int kRA = TM_ / kWaves, kRB = TN_ / kWaves;        // rows a wave fetches per stage
  static constexpr int kATile = TM_ * kRow, kBTile = TN_ * kRow, kStage = kATile + kBTile;
  static_assert(kIM >= 1 && kIN >= 1 && kRA % 16 == 0 && kRB % 16 == 0, "whole 32 x 32 tiles, whole 16-row load blocks");
};
using Mid128 = MidShape<128, 128, 4, 2>;  // 8 waves of 32 x 64, 36 KiB a stage, two workgroups a CU
// One workgroup a CU (or several small ones), for launches of at most one workgroup per CU: the ring schedule.
// (four buffers each: six for the 64 x 64 tile, one workgroup a CU then, measured 23 us where two workgroups a CU
// on four take 16 (512 x 4096 x 4096); five for the others changed nothing)
using Ring128 = MidShape<128, 128, 4, 2, 2, true, 2, true, 4>;
using Ring64x128 = MidShape<64, 128, 2, 2, 2, true, 2, true, 4>;
using Ring64 = MidShape<64, 64, 2, 2, 2, true, 2, true, 4>;
// Eight (six) buffers where a workgroup has its CU to itself, and one barrier per two stages: six (four) stages on
// their way per workgroup.  128 x 4096 x 4096, rows, weight cached / from HBM (a different weight every call):
// 10.0 / 19.8 us on four buffers, 10.3 / 17.1 on eight, 9.4 / 15.6 with the barrier per pair.
using Ring64Pair = MidShape<64, 64, 2, 2, 2, true, 2, true, 8, true>;
using Ring64x128Pair = MidShape<64, 128, 2, 2, 2, true, 2, true, 6, true>;
using Ring128x256 = MidShape<128, 256, 2, 4, 2, true, 1, true, 3>;  // 8 waves of 64 x 64, 144 KiB of LDS

// MMA, EPI, COL_FIRST as in gemm_kernel.  PACKED: a row of B has half the bytes in memory that it has in LDS:
// int4 values two per byte (see gemm_kernel's BPACK), or, with MmaBf16W8, int8 values that become bf16 (A then
// holds bf16 values, and GemmArgs::k, lda and stride_a count its bytes), or, with MmaBf16F8, fp8 bytes that become
// bf16; A's rows are then widened the same way (MMA::kWidenA: GemmArgs::k counts the bf16 bytes of a row in LDS,
// twice the fp8 bytes in memory, while lda and stride_a count those).
// SLAB: this launch writes raw partial sums of a K slice to its slab (EPI is 3 then; integer sums only).
// CONV: A is a convolution input read in place (GemmArgs::conv): the window gather that would otherwise be
// materialised (features % 128 == 0, so a 128-byte stage lies inside one tap).
template <class MMA, int EPI, bool COL_FIRST, bool PACKED, bool SLAB, bool CONV = false, class S = Mid128>
__global__ __launch_bounds__(S::kThreads) __attribute__((amdgpu_waves_per_eu(S::kOcc, S::kOcc)))
void gemm_mid_kernel(const GemmArgs g_in) {
  constexpr int TM = S::kTM, TN = S::kTN, kATile = S::kATile, kStage = S::kStage, kRow = S::kRow;
  constexpr bool SW = S::kSwizzle;
  constexpr int IM = S::kIM, IN = S::kIN, RA = S::kRA, RB = S::kRB;
  constexpr bool RING = S::kRing;
  // ring, swizzled rows, nothing to unpack: pieces go from memory straight into LDS
  constexpr bool DIRECT = RING && SW && !PACKED && !MMA::kWidenA && !CONV && S::kBuffers >= 3;
  constexpr int NB = DIRECT ? S::kBuffers : 0;
  constexpr int NSETS = DIRECT ? 1 : RING ? 3 : 1, NBUF = RING ? 3 : 2;
  static_assert(!CONV || (TM == 128 && S::kWaves == 8), "the window gather is written for two loads of A per wave");
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
  __shared__ __attribute__((aligned(1024))) uint8_t stage_mem[DIRECT ? 16 : NBUF * kStage];
  // the direct ring's buffers are objects of their own, so that the compiler can tell a fragment read of one from
  // a request in flight into another
  __shared__ __attribute__((aligned(1024))) uint8_t ring0[DIRECT ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring1[DIRECT ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring2[DIRECT ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring3[DIRECT && NB > 3 ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring4[DIRECT && NB > 4 ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring5[DIRECT && NB > 5 ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring6[DIRECT && NB > 6 ? kStage : 16];
  __shared__ __attribute__((aligned(1024))) uint8_t ring7[DIRECT && NB > 7 ? kStage : 16];
  static_assert(NB <= 8, "eight ring buffers at most");
  auto ring = [&](const int b) -> uint8_t* {
    return b == 0 ? ring0 : b == 1 ? ring1 : b == 2 ? ring2 : b == 3 ? ring3 : b == 4 ? ring4 : b == 5 ? ring5 : b == 6 ? ring6 : ring7;
  };
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / S::kWN, wn = wave % S::kWN;
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
  constexpr int NLA = WIDEN_A ? RA / 16 : RA / 8, NLB = PACKED ? RB / 16 : RB / 8, NL = NLA + NLB;
  constexpr int kOutside = 0x7FFFFFF0;
  v4i stg[NSETS][NL];
  // A: load j of a wave covers 8 rows x 128 B (16 rows x 64 B of memory where A is widened)
  const int ld_a = WIDEN_A ? (wave * RA + (lane >> 2)) * (int)g.lda + (lane & 3) * 16
                           : (wave * RA + (lane >> 3)) * (int)g.lda + (lane & 7) * 16;
  const int ld_a_next = (WIDEN_A ? 16 : 8) * (int)g.lda;
  // B in fragment order: a wave load is one KiB = 64 bytes of 16 rows (lane -> row lane & 15, bytes 16 (lane >> 4));
  // unpacked, two loads are the two KiB of a 16-row block's stage (the second 64 bytes further in LDS), and the
  // scalar offset advances one KiB per 64 row bytes
  const int ld_b = g.b_frag ? wave * (RB / 16) * g.b_steps * 1024 + lane * 16
                 : PACKED ? (wave * RB + (lane >> 2)) * (int)g.ldb + (lane & 3) * 16
                          : (wave * RB + (lane >> 3)) * (int)g.ldb + (lane & 7) * 16;
  const int kpos_a = WIDEN_A ? (lane & 3) * 32 : (lane & 7) * 16;
  const int kpos_b = g.b_frag ? (lane >> 4) * (PACKED ? 32 : 16) : PACKED ? (lane & 3) * 32 : (lane & 7) * 16;
  // byte offset, within a tile, of 16-byte chunk `chunk` of row `row`
  auto lds_pos = [&](const int row, const int chunk) -> int {
    if constexpr (SW) {
      const int r = row & 31;
      return row * kRow + ((chunk ^ ((r ^ (r >> 3)) & 7)) << 4);
    } else {
      return row * kRow + chunk * 16;
    }
  };
  // where piece j of a stage goes in LDS (the first of its two chunks where a piece is widened to 32 bytes;
  // the second follows it, or, swizzled, is its neighbour under XOR 16)
  int st_off[NL];
#pragma unroll
  for (int j = 0; j < NLA; ++j)
    st_off[j] = WIDEN_A ? lds_pos(wave * RA + j * 16 + (lane >> 2), 2 * (lane & 3))
                        : lds_pos(wave * RA + j * 8 + (lane >> 3), lane & 7);
#pragma unroll
  for (int j = 0; j < NLB; ++j) {
    if constexpr (PACKED)
      st_off[NLA + j] = kATile + (g.b_frag ? lds_pos(wave * RB + j * 16 + (lane & 15), 2 * (lane >> 4))
                                           : lds_pos(wave * RB + j * 16 + (lane >> 2), 2 * (lane & 3)));
    else
      st_off[NLA + j] = kATile + (g.b_frag ? lds_pos(wave * RB + (j >> 1) * 16 + (lane & 15), (lane >> 4) + 4 * (j & 1))
                                           : lds_pos(wave * RB + j * 8 + (lane >> 3), lane & 7));
  }
  constexpr int kSecond = 16;  // second chunk of a widened piece: + 16, or ^ 16 when swizzled
  // load jj of B past the wave's first: memory offset, LDS offset, position along k (jj is a constant where used)
  auto b_mem_next = [&](const int jj) -> int {
    if constexpr (PACKED) return g.b_frag ? jj * g.b_steps * 1024 : jj * 16 * (int)g.ldb;
    else return g.b_frag ? (jj >> 1) * g.b_steps * 1024 + (jj & 1) * 1024 : jj * 8 * (int)g.ldb;
  };
  auto b_kpos_next = [&](const int jj) -> int { return (!PACKED && g.b_frag) ? (jj & 1) * 64 : 0; };
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
  auto load_one = [&](const int set, const int j, int k0) {
    if constexpr (CONV) {
      if (j < NLA) {
        const int d0 = ct0 * g.conv.dil[0], d1 = ct1 * g.conv.dil[1], d2 = ct2 * g.conv.dil[2];
        const bool in = (unsigned)(ci0[j] + d0) < (unsigned)g.conv.in[0] && (unsigned)(ci1[j] + d1) < (unsigned)g.conv.in[1] &&
                        (unsigned)(ci2[j] + d2) < (unsigned)g.conv.in[2] && ct0 < g.conv.ker[0];
        const int tap = ((d0 * g.conv.in[1] + d1) * g.conv.in[2] + d2) * g.conv.c + cch;
        stg[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, in ? cpix[j] + tap + kpos_a : kOutside, 0, 0);
        return;
      }
    }
    if (j < NLA) {
      const int vo = k0 + kpos_a < (int)g.k ? ld_a + j * ld_a_next : kOutside;
      stg[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, vo, WIDEN_A ? k0 / 2 : k0, 0);
    } else if constexpr (PACKED) {
      const int vo = k0 + kpos_b < (int)g.k ? ld_b + b_mem_next(j - NLA) : kOutside;
      stg[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, (k0 / 2) << ksh_b, 0);
    } else {
      const int vo = k0 + kpos_b + b_kpos_next(j - NLA) < (int)g.k ? ld_b + b_mem_next(j - NLA) : kOutside;
      stg[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, k0 << ksh_b, 0);
    }
  };
  auto store_piece = [&](const int set, const int stage_base, const int jj) {
    uint8_t* st = stage_mem + stage_base;
    const int second = SW ? (st_off[jj] ^ kSecond) : st_off[jj] + kSecond;
    if (jj < NLA) {
      if constexpr (WIDEN_A) {
        v4i lo, hi;
        MMA::widen_a(stg[set][jj], lo, hi);
        *reinterpret_cast<v4i*>(st + st_off[jj]) = lo;
        *reinterpret_cast<v4i*>(st + second) = hi;
      } else {
        *reinterpret_cast<v4i*>(st + st_off[jj]) = stg[set][jj];
      }
    } else {
      if constexpr (PACKED) {
        v4i lo, hi;
        if constexpr (MMA::kWidenB) MMA::widen_b(stg[set][jj], lo, hi);
        else unpack_i4x32(stg[set][jj], lo, hi, g.a_even_odd8);
        *reinterpret_cast<v4i*>(st + st_off[jj]) = lo;
        *reinterpret_cast<v4i*>(st + second) = hi;
      } else {
        *reinterpret_cast<v4i*>(st + st_off[jj]) = stg[set][jj];
      }
    }
  };
  auto store_stage = [&](const int set, const int stage_base) {
#pragma unroll
    for (int j = 0; j < NL; ++j) store_piece(set, stage_base, j);
  };

  // fragment of k step ks of a 32-row block: the kChunks chunks from (2 ks + lh) kChunks on of row lr; their
  // offsets within the block are the same for every block (the swizzle looks at the row modulo 32 only)
  constexpr int KS = 4 / kChunks;
  int fo[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) fo[i] = lds_pos(lr, (2 * (i / kChunks) + lh) * kChunks + i % kChunks);
  const int a_blk = wm * 32 * IM * kRow, b_blk = kATile + wn * 32 * IN * kRow;
  // Direct ring with B in fragment order: B keeps that order in LDS (a KiB of memory = 64 bytes of 16 rows is a
  // KiB of LDS: every request is one contiguous KiB; asking for the pieces a swizzled row layout wants instead
  // measured 15.4 against 10.0 us at 128 x 4096 x 4096).  Chunk q of row r of a 32-row block then lies at
  // (2 (r >> 4) + (q >> 2)) KiB + 16 (16 (q & 3) + (r & 15)): the 16 rows of a fragment read are consecutive.
  int fob[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = (2 * (i / kChunks) + lh) * kChunks + i % kChunks;
    fob[i] = (DIRECT && g.b_frag) ? (2 * (lr >> 4) + (q >> 2)) * 1024 + (16 * (q & 3) + (lr & 15)) * 16 : fo[i];
  }
  auto frag_of = [&](const uint8_t* blk, const int ks, const int* off) -> Frag {
    if constexpr (kChunks == 1) {
      return *reinterpret_cast<const v4i*>(blk + off[ks]);
    } else {
      const v4i x0 = *reinterpret_cast<const v4i*>(blk + off[2 * ks]), x1 = *reinterpret_cast<const v4i*>(blk + off[2 * ks + 1]);
      return Frag{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
  };
  auto frag = [&](const uint8_t* blk, const int ks) -> Frag { return frag_of(blk, ks, fo); };
  auto frag_b = [&](const uint8_t* blk, const int ks) -> Frag { return frag_of(blk, ks, fob); };

  Acc acc[IM][IN];
#pragma unroll
  for (int im = 0; im < IM; ++im)
#pragma unroll
    for (int in = 0; in < IN; ++in)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[im][in][r] = 0;

  const int nstages = (int)((g.k + BK - 1) / BK);
  auto lds_barrier = [&]() {  // a bare s_barrier: a __syncthreads() would also wait for the global loads in flight
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  if constexpr (!RING) {
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(0, j, 0);
    if constexpr (CONV) conv_advance();
    store_stage(0, 0);
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(0, j, nstages > 1 ? BK : 0);
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
      for (int ks = 0; ks < KS; ++ks) {
        Frag fa[IM], fb[IN];
#pragma unroll
        for (int im = 0; im < IM; ++im) fa[im] = frag(st + a_blk + im * 32 * kRow, ks);
#pragma unroll
        for (int in = 0; in < IN; ++in) fb[in] = frag_b(st + b_blk + in * 32 * kRow, ks);
#pragma unroll
        for (int im = 0; im < IM; ++im)
#pragma unroll
          for (int in = 0; in < IN; ++in) acc[im][in] = MMA::mma(fb[in], fa[im], acc[im][in]);
      }
      store_stage(0, (1 - BUF) * kStage);
      const int k_next = s + 2 < nstages ? (s + 2) * BK : 0;
#pragma unroll
      for (int j = 0; j < NL; ++j) load_one(0, j, k_next);
      if constexpr (CONV) conv_advance();  // past the last stage the tap leaves the window: zeros nobody reads
      lds_barrier();
    };
    for (int s = 0; s < nstages; s += 2) {
      stage(s, std::integral_constant<int, 0>{});
      if (s + 1 < nstages) stage(s + 1, std::integral_constant<int, 1>{});
    }
  } else if constexpr (DIRECT) {
    // Direct ring: NB LDS buffers, no staging registers and no ds_write (a stage's ds_write_b128, 8 cycles each on
    // the CU's one LDS pipe, added their time whole to the stage).  A piece = 8 rows x 128 B of a wave's share of
    // A or B; lane l asks for the chunk that belongs at position l & 7 of row l >> 3 (chunk (l & 7) ^ f(row)), and
    // the buffer load to LDS puts lane l's 16 bytes at base + 16 l.  Stage s computes from buffer s % NB as in the
    // ring below and, group by group, requests the pieces of stage s + NB - 1 into the buffer stage s - 1 left at
    // its barrier.  Requests complete in order, so before its barrier a wave waits until all but the requests
    // issued after those of stage s + 1 have landed, and behind the barrier everybody's have.
    constexpr int G = S::kGroup, NG = KS / G, D = NB - 1;
    static_assert(NG >= 2 && NG % 2 == 0, "the last group computes from fragment set 1");
    static_assert(NLA == RA / 8 && NLB == RB / 8, "pieces of 8 rows");
    static_assert(RB % 16 == 0, "a wave's share of fragment-ordered B is whole 16-row blocks");
    auto k_of = [&](const int s) -> int { return s < nstages ? s * BK : 0; };
    int dvo[NL], dkp[NL];  // vector offset of a piece's request and its position along k (for the mask on K)
#pragma unroll
    for (int j = 0; j < NL; ++j) {
      const bool is_b = j >= NLA;
      const int row = is_b ? wave * RB + (j - NLA) * 8 + (lane >> 3) : wave * RA + j * 8 + (lane >> 3);
      const int r = row & 31;
      const int c = (lane & 7) ^ ((r ^ (r >> 3)) & 7);
      dkp[j] = c * 16;
      dvo[j] = !is_b ? row * (int)g.lda + c * 16 : row * (int)g.ldb + c * 16;
      if (is_b && g.b_frag) {
        // piece jj = half (jj & 1) of the stage of 16-row block wave * RB / 16 + (jj >> 1): one KiB of memory
        const int jj = j - NLA;
        dvo[j] = ((wave * (RB / 16) + (jj >> 1)) * g.b_steps + (jj & 1)) * 1024 + lane * 16;
        dkp[j] = (jj & 1) * 64 + (lane >> 4) * 16;
      }
    }
    auto request = [&](uint8_t* buf, const int j, const int k0) {
      const int vo = k0 + dkp[j] < (int)g.k ? dvo[j] : kOutside;
      if (j < NLA)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(buf + (wave * RA + j * 8) * kRow), 16, vo, k0, 0, 0);
      else
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)(buf + kATile + (wave * RB + (j - NLA) * 8) * kRow), 16, vo, k0 << ksh_b, 0, 0);
    };
    Frag fa[2][G][IM], fb[2][G][IN];
    auto load_frags = [&](const uint8_t* st, const int gi, const int fs) {
#pragma unroll
      for (int q = 0; q < G; ++q) {
#pragma unroll
        for (int im = 0; im < IM; ++im) fa[fs][q][im] = frag(st + a_blk + im * 32 * kRow, gi * G + q);
#pragma unroll
        for (int in = 0; in < IN; ++in) fb[fs][q][in] = frag_b(st + b_blk + in * 32 * kRow, gi * G + q);
      }
    };
    auto mfma_group = [&](const int fs) {
#pragma unroll
      for (int q = 0; q < G; ++q)
#pragma unroll
        for (int im = 0; im < IM; ++im)
#pragma unroll
          for (int in = 0; in < IN; ++in) acc[im][in] = MMA::mma(fb[fs][q][in], fa[fs][q][im], acc[im][in]);
    };
    if constexpr (S::kPair) {
      // Two stages per barrier.  A 64 x 64 tile gives each of its four waves four matrix instructions a stage, and
      // the wait, the barrier and the latency of the first fragment reads behind it cost more than those; here a
      // wave waits and meets the others once per 256 bytes of k.  Stages 2 S and 2 S + 1 are computed group by
      // group as one stage of 2 NG groups, and their share of the requests is the two stages NB - 2 ahead, into
      // the two buffers that the previous pair left at its barrier.  Stages past the end of k are requested like
      // any other: the mask on k makes them zeros, so an odd stage count needs no special case.
      static_assert(NB % 2 == 0 && NB >= 6, "pairs of buffers, and a pair's requests have a pair to land");
      constexpr int D2 = NB - 2, NG2 = 2 * NG, NL2 = 2 * NL;
      auto k_at = [&](const int s) -> int { return s * BK; };
#pragma unroll
      for (int d = 0; d < D2; ++d)
#pragma unroll
        for (int j = 0; j < NL; ++j) request(ring(d), j, k_at(d));
      asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D2 - 2) * NL) : "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      load_frags(ring0, 0, 0);
      constexpr int kBefore2 = (NG2 - 1) * NL2 / NG2;
      constexpr int kAfterNext2 = (D2 - 4) * NL + kBefore2;  // requests issued after those of the next pair
      static_assert(kAfterNext2 <= 63, "vmcnt");
      auto pair_stage = [&](const int s, auto buf_c) {
        constexpr int B0 = decltype(buf_c)::value, W0 = (B0 + D2) % NB, N0 = (B0 + 2) % NB;
        const int k_req0 = k_at(s + D2), k_req1 = k_at(s + D2 + 1);
        auto refill = [&](const int gi) {
#pragma unroll
          for (int j = gi * NL2 / NG2; j < (gi + 1) * NL2 / NG2; ++j) {
            if (j < NL) request(ring(W0), j, k_req0);
            else request(ring(W0 + 1), j - NL, k_req1);
          }
        };
#pragma unroll
        for (int gi = 0; gi < NG2 - 1; ++gi) {
          load_frags(ring(B0 + (gi + 1) / NG), (gi + 1) % NG, (gi + 1) & 1);
          refill(gi);
          mfma_group(gi & 1);
        }
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kAfterNext2) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        mfma_group(1);
        load_frags(ring(N0), 0, 0);
        refill(NG2 - 1);
      };
      for (int s = 0; s < nstages; s += NB) {
        pair_stage(s, std::integral_constant<int, 0>{});
        if (s + 2 < nstages) pair_stage(s + 2, std::integral_constant<int, 2>{});
        if (s + 4 < nstages) pair_stage(s + 4, std::integral_constant<int, 4>{});
        if constexpr (NB > 6) {
          if (s + 6 < nstages) pair_stage(s + 6, std::integral_constant<int, 6>{});
        }
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    } else {
#pragma unroll
    for (int d = 0; d < D; ++d)
#pragma unroll
      for (int j = 0; j < NL; ++j) request(ring(d), j, k_of(d));
    // stage 0 has landed when at most the requests of stages 1 .. D - 1 are outstanding
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"((D - 1) * NL) : "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    load_frags(ring0, 0, 0);
    constexpr int kBefore = (NG - 1) * NL / NG;              // pieces a stage requests before its barrier
    constexpr int kAfterNext = (D - 2) * NL + kBefore;       // requests issued after those of the next stage
    static_assert(kAfterNext <= 63, "vmcnt");
    auto stage = [&](const int s, auto buf_c) {
      constexpr int BUF = decltype(buf_c)::value, W = (BUF + D) % NB, NXT = (BUF + 1) % NB;
      const uint8_t* cur = ring(BUF);
      const uint8_t* next = ring(NXT);
      const int k_req = k_of(s + D);
      auto refill = [&](const int gi) {
#pragma unroll
        for (int j = gi * NL / NG; j < (gi + 1) * NL / NG; ++j) request(ring(W), j, k_req);
      };
#pragma unroll
      for (int gi = 0; gi < NG - 1; ++gi) {
        load_frags(cur, gi + 1, (gi + 1) & 1);
        refill(gi);
        mfma_group(gi & 1);
      }
      asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(kAfterNext) : "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      mfma_group(1);
      load_frags(next, 0, 0);
      refill(NG - 1);
    };
    for (int s = 0; s < nstages; s += NB) {
      stage(s, std::integral_constant<int, 0>{});
      if (s + 1 < nstages) stage(s + 1, std::integral_constant<int, 1>{});
      if (s + 2 < nstages) stage(s + 2, std::integral_constant<int, 2>{});
      if constexpr (NB > 3) {
        if (s + 3 < nstages) stage(s + 3, std::integral_constant<int, 3>{});
      }
      if constexpr (NB > 4) {
        if (s + 4 < nstages) stage(s + 4, std::integral_constant<int, 4>{});
      }
      if constexpr (NB > 5) {
        if (s + 5 < nstages) stage(s + 5, std::integral_constant<int, 5>{});
      }
      if constexpr (NB > 6) {
        if (s + 6 < nstages) stage(s + 6, std::integral_constant<int, 6>{});
      }
      if constexpr (NB > 7) {
        if (s + 7 < nstages) stage(s + 7, std::integral_constant<int, 7>{});
      }
    }
    // requests past the end of k (they repeat stage 0) have to land before the epilogue stages the output in the
    // same buffers
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
  } else {
    // Ring schedule: three LDS buffers, three staging sets.  Stage s computes from buffer s % 3, group by group
    // (a group = kGroup k steps whose fragments are read together, one group ahead of the matrix instructions
    // that use them).  Its share of every group: a piece of stage s + 2 goes from staging set (s + 2) % 3 to
    // buffer (s + 2) % 3 (free since the barrier of stage s - 1: it held stage s - 1) and the same piece of stage
    // s + 5 is requested into the registers just emptied, so that LDS writes and memory requests are spread over
    // the stage and a request has three stages to arrive.  The barrier stands before the last group: every wave
    // then holds its last fragments of stage s, and everything of stage s + 1 (written during stage s - 1) is
    // published, so the first fragments of stage s + 1 are read under the last group's matrix instructions.
    constexpr int G = S::kGroup, NG = KS / G;
    static_assert(NG >= 2 && NG % 2 == 0, "the last group computes from fragment set 1");
    static_assert(!CONV, "requests would have to advance the window tap piece by piece");
    auto k_of = [&](const int s) -> int { return s < nstages ? s * BK : 0; };
    Frag fa[2][G][IM], fb[2][G][IN];
    auto load_frags = [&](const uint8_t* st, const int gi, const int fs) {
#pragma unroll
      for (int q = 0; q < G; ++q) {
#pragma unroll
        for (int im = 0; im < IM; ++im) fa[fs][q][im] = frag(st + a_blk + im * 32 * kRow, gi * G + q);
#pragma unroll
        for (int in = 0; in < IN; ++in) fb[fs][q][in] = frag_b(st + b_blk + in * 32 * kRow, gi * G + q);
      }
    };
    auto mfma_group = [&](const int fs) {
#pragma unroll
      for (int q = 0; q < G; ++q)
#pragma unroll
        for (int im = 0; im < IM; ++im)
#pragma unroll
          for (int in = 0; in < IN; ++in) acc[im][in] = MMA::mma(fb[fs][q][in], fa[fs][q][im], acc[im][in]);
    };
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(0, j, k_of(0));
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(1, j, k_of(1));
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(2, j, k_of(2));
    store_stage(0, 0);
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(0, j, k_of(3));
    store_stage(1, kStage);
#pragma unroll
    for (int j = 0; j < NL; ++j) load_one(1, j, k_of(4));
    lds_barrier();
    load_frags(stage_mem, 0, 0);
    auto stage = [&](const int s, auto buf_c) {
      constexpr int BUF = decltype(buf_c)::value, W = (BUF + 2) % 3, NXT = (BUF + 1) % 3;
      const uint8_t* cur = stage_mem + BUF * kStage;
      const uint8_t* next = stage_mem + NXT * kStage;
      const int k_req = k_of(s + 5);
      auto refill = [&](const int gi) {
#pragma unroll
        for (int j = gi * NL / NG; j < (gi + 1) * NL / NG; ++j) {
          store_piece(W, W * kStage, j);
          load_one(W, j, k_req);
        }
      };
#pragma unroll
      for (int gi = 0; gi < NG - 1; ++gi) {
        load_frags(cur, gi + 1, (gi + 1) & 1);
        refill(gi);
        mfma_group(gi & 1);
      }
      lds_barrier();
      mfma_group(1);
      load_frags(next, 0, 0);
      refill(NG - 1);
    };
    for (int s = 0; s < nstages; s += 3) {
      stage(s, std::integral_constant<int, 0>{});
      if (s + 1 < nstages) stage(s + 1, std::integral_constant<int, 1>{});
      if (s + 2 < nstages) stage(s + 2, std::integral_constant<int, 2>{});
    }
  }

  // ---- epilogue: lane holds C[m = wm*32*IM + im*32 + lr][n = wn*32*IN + ni*32 + 8q + 4lh + e], register 4q + e of tile (im, ni)
  // Where rows of C start 16-byte aligned, a wave passes its part of the tile through LDS (a region of its own
  // in the stage buffers, which nobody reads any more) so that the stores are 16 bytes a lane along whole row
  // segments: straight from the accumulator layout a store instruction touches 16 bytes in each of 32 rows.
  if constexpr (!SLAB) {
    constexpr bool kOutBf16 = EPI <= 1 || EPI == 4;
    constexpr int kEsz = kOutBf16 ? 2 : 4;
    constexpr int kRowBytes = 32 * IN * kEsz, kPitch = kRowBytes + 16, kWaveBytes = 32 * IM * kPitch;
    // (direct ring: the waves share out its buffers, wave w in buffer w % NB)
    constexpr bool kStagedFits = DIRECT ? ((S::kWaves + NB - 1) / (DIRECT ? NB : 1)) * kWaveBytes <= kStage
                                        : S::kWaves * kWaveBytes <= NBUF * kStage;
    static_assert(DIRECT || kStagedFits, "the staged tile fits the stage buffers");
    const bool staged = kStagedFits && g.acc_out == nullptr && ((g.ldc * kEsz) % 16) == 0 && ((g.stride_c * kEsz) % 16) == 0 &&
                        ((uintptr_t)g.c % 16) == 0 && ((n0 * kEsz) % 16) == 0;
    if (staged) {
      lds_barrier();
      uint8_t* mine = DIRECT ? ring(wave % (DIRECT ? NB : 1)) + (wave / (DIRECT ? NB : 1)) * kWaveBytes : stage_mem + wave * kWaveBytes;
      const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
      const bool cs_vec = ((uintptr_t)cs % 16) == 0;
#pragma unroll
      for (int im = 0; im < IM; ++im) {
        const int64_t mm = m0 + wm * 32 * IM + im * 32 + lr;
        const float s_row = (g.row_scale && mm < g.m) ? g.row_scale[bz * g.stride_rs + mm] : 1.0f;
#pragma unroll
        for (int ni = 0; ni < IN; ++ni)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int col = ni * 32 + 8 * q + 4 * lh;
            const int64_t nn = n0 + wn * 32 * IN + col;
            AccScalar v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              if constexpr (PACKED && MMA::kIntAcc) v[e] = acc[im][ni][4 * q + e] >> 4;
              else v[e] = acc[im][ni][4 * q + e];
            }
            uint8_t* at = mine + (im * 32 + lr) * kPitch + col * kEsz;
            if constexpr (EPI == 3) {
              *reinterpret_cast<int4*>(at) = make_int4(v[0], v[1], v[2], v[3]);
            } else {
              float csv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
              if (cs != nullptr) {
                if (nn + 4 <= g.n && cs_vec) {
                  const float4 c4 = *reinterpret_cast<const float4*>(cs + nn);
                  csv[0] = c4.x; csv[1] = c4.y; csv[2] = c4.z; csv[3] = c4.w;
                } else {
                  for (int e = 0; e < 4 && nn + e < g.n; ++e) csv[e] = cs[nn + e];
                }
              }
              float o[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = dequant_value<EPI, COL_FIRST>(v[e], s_row, csv[e]);
              if constexpr (kOutBf16) {
                uint2 w;
                w.x = (uint32_t)bf16_bits(o[0]) | ((uint32_t)bf16_bits(o[1]) << 16);
                w.y = (uint32_t)bf16_bits(o[2]) | ((uint32_t)bf16_bits(o[3]) << 16);
                *reinterpret_cast<uint2*>(at) = w;
              } else {
                *reinterpret_cast<float4*>(at) = make_float4(o[0], o[1], o[2], o[3]);
              }
            }
          }
      }
      // the wave's own stores, in order with its reads below: no barrier
      constexpr int kLanesPerRow = kRowBytes / 16, kRowsPerPass = 64 / kLanesPerRow, kPerLane = 16 / kEsz;
      const int pr = lane / kLanesPerRow, pc = lane % kLanesPerRow;
#pragma unroll
      for (int it = 0; it < 32 * IM / kRowsPerPass; ++it) {
        const int r = it * kRowsPerPass + pr;
        const v4i val = *reinterpret_cast<const v4i*>(mine + r * kPitch + pc * 16);
        const int64_t mm = m0 + wm * 32 * IM + r;
        const int64_t nn = n0 + wn * 32 * IN + pc * kPerLane;
        if (mm >= g.m || nn >= g.n) continue;
        uint8_t* dst = reinterpret_cast<uint8_t*>(g.c) + (bz * g.stride_c + mm * g.ldc + nn) * kEsz;
        if (nn + kPerLane <= g.n) {
          *reinterpret_cast<v4i*>(dst) = val;
        } else {
          for (int e = 0; e < kPerLane && nn + e < g.n; ++e) {
            if constexpr (kEsz == 2) reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)((uint32_t)val[e >> 1] >> (16 * (e & 1)));
            else reinterpret_cast<int32_t*>(dst)[e] = val[e];
          }
        }
      }
      return;
    }
  }
#pragma unroll
  for (int im = 0; im < IM; ++im) {
    const int64_t mm = m0 + wm * 32 * IM + im * 32 + lr;
    if (mm >= g.m) continue;
    if constexpr (SLAB) {
      int32_t* dst = g.slabs + (((int64_t)blockIdx.z * gridDim.y + bz) * g.m + mm) * g.n;
      const bool vec = (g.n % 4) == 0;
#pragma unroll
      for (int ni = 0; ni < IN; ++ni)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t nn = n0 + wn * 32 * IN + ni * 32 + 8 * q + 4 * lh;
          if (nn >= g.n) continue;
          int v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = PACKED ? acc[im][ni][4 * q + e] >> 4 : acc[im][ni][4 * q + e];  // exact: multiples of 16 (SLAB: int4)
          if (vec) *reinterpret_cast<int4*>(dst + nn) = make_int4(v[0], v[1], v[2], v[3]);
          else for (int e = 0; e < 4 && nn + e < g.n; ++e) dst[nn + e] = v[e];
        }
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
      for (int ni = 0; ni < IN; ++ni)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int64_t nn = n0 + wn * 32 * IN + ni * 32 + 8 * q + 4 * lh;
          if (nn >= g.n) continue;
          const bool full = nn + 4 <= g.n;
          AccScalar v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (PACKED && MMA::kIntAcc) v[e] = acc[im][ni][4 * q + e] >> 4;
            else v[e] = acc[im][ni][4 * q + e];
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
}

template <int EPI, bool COL_FIRST, class S = Mid128>
void launch_mid(const GemmArgs& g, bool packed, dim3 grid, hipStream_t st) {
  if constexpr (!COL_FIRST) {
    if (packed) { gemm_mid_kernel<MmaI8, EPI, false, true, false, false, S><<<grid, S::kThreads, 0, st>>>(g); return; }
  }
  gemm_mid_kernel<MmaI8, EPI, COL_FIRST, false, false, false, S><<<grid, S::kThreads, 0, st>>>(g);
}

// Every epilogue of the int8 contraction on tile shape S.
template <class S>
void launch_mid_shape(GemmArgs g, const aqtx_gemm_plan* p, int epi, bool packed, hipStream_t st) {
  g.tiles_m = (int)((p->m + S::kTM - 1) / S::kTM);
  g.tiles_n = (int)((p->n + S::kTN - 1) / S::kTN);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  switch (epi) {
    case 0: if (g.col_first) launch_mid<0, true, S>(g, packed, grid, st); else launch_mid<0, false, S>(g, packed, grid, st); break;
    case 1: if (g.col_first) launch_mid<1, true, S>(g, packed, grid, st); else launch_mid<1, false, S>(g, packed, grid, st); break;
    case 2: if (g.col_first) launch_mid<2, true, S>(g, packed, grid, st); else launch_mid<2, false, S>(g, packed, grid, st); break;
    case 4: if (g.col_first) launch_mid<4, true, S>(g, packed, grid, st); else launch_mid<4, false, S>(g, packed, grid, st); break;
    default: launch_mid<3, false, S>(g, packed, grid, st); break;
  }
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

// Tile shape for a plan on `cus` CUs (plan->tuning values).  At most one 128 x 128 tile per CU: the ring
// schedule (a workgroup alone on its CU has nobody to overlap its waits with: the ring hides them itself), on
// the smallest tiles that still give every workgroup a CU to itself: 64 x 64 on eight buffers, else 64 x 128 on
// six, both with one barrier per two stages (512 x 4096 x 4096, weight cached / from HBM: 16.6 / 20.5 us on the
// latter against 16.6 / 22.4 on 64 x 64 tiles, four buffers, two workgroups a CU), on 128 x 128 tiles beyond.  More than one 128 x 128 tile but at most one 128 x 256 tile per CU: the ring on
// those.  Beyond: 128 x 128 tiles on the plain schedule, two workgroups a CU.
inline int mid_shape_for(const aqtx_gemm_plan* p, int cus) {
  const int64_t tiles128 = ((p->m + 127) / 128) * ((p->n + 127) / 128) * p->batch;
  const int64_t tiles256 = ((p->m + 127) / 128) * ((p->n + 255) / 256) * p->batch;
  // (not for a k of fewer than eight stages: the ring's five stages of lead are most of such a tile;
  // 4096 x 2048 x 512 measured 15.5 us on it against 13.9 us on the plain schedule)
  if (tiles128 > cus) return (tiles256 <= cus && p->k >= 1024) ? 132 : 128;
  const int64_t tiles64 = ((p->m + 63) / 64) * ((p->n + 63) / 64) * p->batch;
  const int64_t tiles64x128 = ((p->m + 63) / 64) * ((p->n + 127) / 128) * p->batch;
  return tiles64 <= cus ? 133 : tiles64x128 <= cus ? 134 : 129;
}

template <class S>
void launch_weight_only_shape(GemmArgs g, const aqtx_gemm_plan* p, hipStream_t st) {
  g.tiles_m = (int)((p->m + S::kTM - 1) / S::kTM);
  g.tiles_n = (int)((p->n + S::kTN - 1) / S::kTN);
  const dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  if (p->col_scale_dtype == AQTX_BF16) gemm_mid_kernel<MmaBf16W8, 0, false, true, false, false, S><<<grid, S::kThreads, 0, st>>>(g);
  else gemm_mid_kernel<MmaBf16W8, 4, false, true, false, false, S><<<grid, S::kThreads, 0, st>>>(g);
}

template <int EPI>
void launch_slab_sum(const GemmArgs& g, dim3 grid, hipStream_t st) {
  if constexpr (EPI != 3) {
    if (g.col_first) { dequant_slabs_kernel<EPI, true><<<grid, 256, 0, st>>>(g); return; }
  }
  dequant_slabs_kernel<EPI, false><<<grid, 256, 0, st>>>(g);
}

}  // namespace

// Whether the kernel of this file takes the plan (0 = no) and in how many slices of K (1 = none).
// plan->tuning: 128 = the 128 x 128 tiles on the plain schedule, 129 | 130 | 131 | 132 | 133 | 134 = the ring schedule
// on 128 x 128 | 64 x 128 | 64 x 64 | 128 x 256 | 64 x 64 (eight buffers, a barrier per two stages) | 64 x 128 (six
// buffers, the same) tiles (in slices only where plan->k_split asks for them, and only unpacked operands).
int gemm_mid_k_slices(const aqtx_gemm_plan* p) {
  if (p->group_offsets != nullptr || (p->tuning != 0 && (p->tuning < 128 || p->tuning > 134)) || !gemm_vector_shape_ok(p)) return 0;  // 4, 8, 16: the large tiles
  if (p->b_dtype == AQTX_I4P && p->scale_order != AQTX_SCALE_ROW_THEN_COL) return 0;
  if (p->lda * (int64_t)TM >= (1ll << 31) || p->ldb * (int64_t)(2 * TN) >= (1ll << 31)) return 0;  // 32-bit offsets within a tile of up to 128 x 256
  const int64_t pad256 = ((p->m + BM - 1) / BM) * ((p->n + BN - 1) / BN);
  const int64_t pad128 = ((p->m + TM - 1) / TM) * ((p->n + TN - 1) / TN);
  const int64_t tiles256 = pad256 * p->batch, tiles128 = pad128 * p->batch;
  const int64_t max_by_k = (p->k + 2 * BK - 1) / (2 * BK);  // a slice holds at least two stages
  if (p->tuning > 128 && !(p->k_split > 1 && p->b_dtype != AQTX_I4P)) return 1;
  if (p->k_split > 1) return (int)(p->k_split < max_by_k ? p->k_split : max_by_k);
  // the large tiles fill the chip, unless a third of their area or more lies outside C (n or m of 128, say)
  const bool padded = 4 * pad256 * 2 >= 3 * pad128;
  if (p->tuning < 128 && tiles256 > 128 && !padded) return 0;
  if (p->k_split == 1 || tiles256 > 128) return 1;
  // A long k over few tiles (half the CUs or fewer): slices until about 256 workgroups exist, each
  // walking at least 1024 of k; the slabs they write and the sum kernel reads stay small next to the operands
  // at such tile counts.  Measured at 4096 columns: k = 14336 in 23 us (128 rows) and 32 us (256 rows) against
  // 35 and 36 us for the smaller tiles of the ring schedule on all of k, and at 512 rows two slices in 50.5 us
  // against 51 (58 against 74 us when the weight comes from HBM); k = 4096 in 17.5 and 20 us against 10 and 11 us
  // (19.5 and 21 against 17 from HBM), so a k below 8192 is never cut.
  if (p->k < 8192 || 2 * tiles128 > 256) return 1;
  // Unpacked operands, k below 10240, and the ring's deep shapes (64 x 64 tiles, or 64 x 128 beyond 256 of those)
  // would put a workgroup on more than half of 256 CUs: no slices.  Measured at 4096 columns, k = 8192, weight
  // cached / from HBM: 256 rows 18.7 / 25.2 us against 23.9 / 27.0 in four slices, 512 rows 28.0 / 36.6 against
  // 35.0 / 37.6 in two; but 128 rows (128 tiles) 17.7 / 24.9 against 19.0 / 20.7 in eight, and at k = 11008 and
  // beyond the slices are ahead from HBM (256 rows: 30.9 against 33.1 us; k = 14336: 34.9 against 41.5).
  if (p->k < 10240 && p->b_dtype != AQTX_I4P) {
    const int64_t tiles64 = ((p->m + 63) / 64) * ((p->n + 63) / 64) * p->batch;
    const int64_t ring_tiles = tiles64 <= 256 ? tiles64 : ((p->m + 63) / 64) * ((p->n + 127) / 128) * p->batch;
    if (ring_tiles <= 256 && 2 * ring_tiles > 256) return 1;
  }
  int64_t s = 256 / tiles128;
  if (s > 8) s = 8;
  // unpacked operands, up to 64 tiles of 64 x 128: the slices run on those, e.g. four instead of eight on
  // 128 x 128 (128 x 4096 x 14336, weight cached / from HBM: 20.8 / 26.8 us against 23.3 / 26.7; k = 8192:
  // 16.3 / 19.2 against 18.9 / 20.8)
  const int64_t tiles64x128 = ((p->m + 63) / 64) * ((p->n + 127) / 128) * p->batch;
  if (p->b_dtype != AQTX_I4P && 4 * tiles64x128 <= 256) s = 256 / tiles64x128 < 8 ? 256 / tiles64x128 : 8;
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
    auto ring_slices = [&](auto shape_tag) {
      using SH = decltype(shape_tag);
      g.tiles_m = (int)((p->m + SH::kTM - 1) / SH::kTM);
      g.tiles_n = (int)((p->n + SH::kTN - 1) / SH::kTN);
      const dim3 rgrid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch, (unsigned)g.k_split);
      gemm_mid_kernel<MmaI8, 3, false, false, true, false, SH><<<rgrid, SH::kThreads, 0, st>>>(g);
    };
    // Unpacked operands: the slices run on the ring, its pieces requested straight into LDS, wherever that puts at
    // most one workgroup on a CU (the plain schedule alone on its CU spends 1300 cycles on a stage's 512 cycles of
    // matrix instructions): 64 x 128 tiles while they fit, else 128 x 128.  512 x 4096 x 14336 in two slices, weight
    // cached / from HBM: 45.4 / 54.3 us against 49.8 / 57.5 on the plain schedule; 256 rows in four: 29.1 / 34.8
    // against 31.2 / 35.2.
    const int cus = compute_units();
    const int64_t wg64x128 = ((p->m + 63) / 64) * ((p->n + 127) / 128) * p->batch * g.k_split;
    const int64_t wg128 = (int64_t)g.tiles_m * g.tiles_n * p->batch * g.k_split;
    if (packed) gemm_mid_kernel<MmaI8, 3, false, true, true><<<grid, 512, 0, st>>>(g);
    else if (p->tuning == 129) ring_slices(Ring128{});
    else if (p->tuning == 133) ring_slices(Ring64Pair{});
    else if (p->tuning == 134) ring_slices(Ring64x128Pair{});
    else if (p->tuning == 0 && wg64x128 <= cus) ring_slices(Ring64x128Pair{});
    else if (p->tuning == 0 && wg128 <= cus) ring_slices(Ring128{});
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
  // tile shape: plan->tuning 128 .. 131 names one (tests, measurements)
  const int shape = p->tuning >= 128 ? p->tuning : mid_shape_for(p, compute_units());
  switch (shape) {
    case 132: launch_mid_shape<Ring128x256>(g, p, epi, packed, st); break;
    case 133: launch_mid_shape<Ring64Pair>(g, p, epi, packed, st); break;
    case 134: launch_mid_shape<Ring64x128Pair>(g, p, epi, packed, st); break;
    case 129: launch_mid_shape<Ring128>(g, p, epi, packed, st); break;
    case 130: launch_mid_shape<Ring64x128>(g, p, epi, packed, st); break;
    case 131: launch_mid_shape<Ring64>(g, p, epi, packed, st); break;
    default: launch_mid_shape<Mid128>(g, p, epi, packed, st); break;
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
  // (the widened weight goes through registers, where the deeper rings change nothing: their tile counts choose
  // the same tiles on the three-buffer ring, 64 x 64 up to half a 128 x 128 tile per CU)
  int shape = p->tuning >= 128 ? p->tuning : mid_shape_for(p, compute_units());
  if (p->tuning == 0 && shape == 134) {
    const int64_t tiles128 = ((p->m + 127) / 128) * ((p->n + 127) / 128) * p->batch;
    shape = 2 * tiles128 <= compute_units() ? 131 : 129;
  }
  switch (shape) {
    case 132: launch_weight_only_shape<Ring128x256>(g, p, st); break;
    case 129: launch_weight_only_shape<Ring128>(g, p, st); break;
    case 130: case 134: launch_weight_only_shape<Ring64x128>(g, p, st); break;
    case 131: case 133: launch_weight_only_shape<Ring64>(g, p, st); break;
    default: launch_weight_only_shape<Mid128>(g, p, st); break;
  }
  AQTX_HIP_CHECK_LAUNCH("gemm_mid_kernel<weight only>");
  return 0;
}

}  // namespace aqtx

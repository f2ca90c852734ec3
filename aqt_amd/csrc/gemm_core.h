// Tiled MFMA contraction with the dequantisation fused in the epilogue, shared by the
// int8 and the fp8 entry points (the element type only changes the MFMA instruction,
// the fragment width and the accumulator type).
//
// C[m, n] = dequant( sum_k A[m, k] * B[n, k] ): both operands carry the
// contraction axis contiguously (the quantize kernels write whichever layout the
// consumer needs), so every lane feeds the MFMA with 16 (int8) or 32 (fp8)
// contiguous bytes per operand.
//
// Tiling: one workgroup (4 waves, 2x2) owns a 256x256 tile of C; a wave owns
// 128x128 = 4x4 MFMA tiles (256 accumulator registers).  K advances 128 bytes per
// stage; two LDS stages of (256+256) rows x 128 B are filled from registers while
// the MFMAs of the other stage run.  Rows are 128 B apart in LDS, so the 16-byte
// chunk index is XOR-swizzled with (row ^ row>>3) & 7: the 16-lane groups of a
// ds_read_b128/ds_write_b128 then touch 64 distinct banks.
//
// The MFMA "A" operand is fed from the B tile and vice versa, so a lane ends up
// holding 4 consecutive n for one m; the epilogue converts, scales, packs these
// and sends them through LDS to leave as full 256-byte row segments.
#pragma once
#include <type_traits>

#include "common.h"

namespace aqtx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v16f __attribute__((ext_vector_type(16)));

// Element traits.  `mma(x, y, c)` computes c += x * y^T for two 32-row fragments; a fragment
// holds kChunks 16-byte chunks per lane (lane>>5 selects the k half inside one MFMA).
struct MmaI8 {
  using Acc = v16i;
  using AccScalar = int32_t;
  using Frag = v4i;
  static constexpr int kChunks = 1;   // v_mfma_i32_32x32x32_i8: 32 k per MFMA, 16 per lane
  static constexpr bool kIntAcc = true;
  static constexpr bool kWidenA = false, kWidenB = false;
  static __device__ __forceinline__ Acc mma(const Frag& x, const Frag& y, const Acc& c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(x, y, c, 0, 0, 0);
  }
  static __device__ __forceinline__ float decode(uint8_t v) { return (float)(int8_t)v; }
};

// FMT_A / FMT_B: 0 = e4m3fn, 1 = e5m2 for the operand holding the rows of C (A) and the
// columns of C (B).  v_mfma_scale_f32_32x32x64_f8f6f4 with both block scales at 2^0.
template <int FMT_A, int FMT_B>
struct MmaF8 {
  using Acc = v16f;
  using AccScalar = float;
  using Frag = v8i;
  static constexpr int kChunks = 2;   // 64 k per MFMA, 32 per lane
  static constexpr bool kIntAcc = false;
  static constexpr bool kWidenA = false, kWidenB = false;
  // x comes from the B tile, y from the A tile (see mfma_step).  Zero scale operands select the
  // unscaled form of the instruction (v_mfma_f32_32x32x64_f8f6f4).
  static __device__ __forceinline__ Acc mma(const Frag& x, const Frag& y, const Acc& c) {
    return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(x, y, c, FMT_B, FMT_A, 0, 0, 0, 0);
  }
};

// Weight-only contraction: A holds bf16 values, B int8 values that are widened to bf16 (exactly) on their
// way to LDS, where both tiles then hold 16-byte chunks of 8 bf16.  v_mfma_f32_32x32x16_bf16, float sums.
struct MmaBf16W8 {
  typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
  using Acc = v16f;
  using AccScalar = float;
  using Frag = v4i;
  static constexpr int kChunks = 1;   // 16 k per MFMA, 8 per lane: 16 bytes
  static constexpr bool kIntAcc = false;
  static constexpr bool kWidenA = false, kWidenB = true;
  static __device__ __forceinline__ Acc mma(const Frag& x, const Frag& y, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, x), __builtin_bit_cast(v8bf, y), c, 0, 0, 0);
  }
  // 16 int8 values (k order) -> 16 bf16 values in two 16-byte chunks.  Every int8 value is a bf16 value, so
  // the upper half of its float32 form is the result.
  static __device__ __forceinline__ void widen_b(const v4i x4, v4i& lo, v4i& hi) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const int x = x4[d];
      const uint32_t f0 = __float_as_uint((float)(int8_t)x), f1 = __float_as_uint((float)(int8_t)(x >> 8));
      const uint32_t f2 = __float_as_uint((float)(int8_t)(x >> 16)), f3 = __float_as_uint((float)(x >> 24));
      const int w0 = (int)__builtin_amdgcn_perm(f1, f0, 0x07060302u), w1 = (int)__builtin_amdgcn_perm(f3, f2, 0x07060302u);
      if (d < 2) { lo[2 * d] = w0; lo[2 * d + 1] = w1; }
      else { hi[2 * (d - 2)] = w0; hi[2 * (d - 2) + 1] = w1; }
    }
  }
};

// 16 fp8 bytes (FMT 0 = e4m3fn, 1 = e5m2; k order) -> 16 bf16 values in two 16-byte chunks.  Every fp8 value,
// subnormals included, is a bf16 value (3 or 2 mantissa bits against 7, a narrower exponent range), so the upper
// half of its float32 form is the result; a NaN byte stays a NaN.
template <int FMT>
__device__ __forceinline__ void widen_f8x16_bf16(const v4i x4, v4i& lo, v4i& hi) {
  typedef float v2f __attribute__((ext_vector_type(2)));
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int x = x4[d];
    const v2f p0 = FMT ? __builtin_amdgcn_cvt_pk_f32_bf8(x, false) : __builtin_amdgcn_cvt_pk_f32_fp8(x, false);
    const v2f p1 = FMT ? __builtin_amdgcn_cvt_pk_f32_bf8(x, true) : __builtin_amdgcn_cvt_pk_f32_fp8(x, true);
    const int w0 = (int)__builtin_amdgcn_perm(__float_as_uint(p0[1]), __float_as_uint(p0[0]), 0x07060302u);
    const int w1 = (int)__builtin_amdgcn_perm(__float_as_uint(p1[1]), __float_as_uint(p1[0]), 0x07060302u);
    if (d < 2) { lo[2 * d] = w0; lo[2 * d + 1] = w1; }
    else { hi[2 * (d - 2)] = w0; hi[2 * (d - 2) + 1] = w1; }
  }
}

// fp8 x fp8 with float32-like sums (aqtx_gemm_plan.accumulate = AQTX_ACC_F32): both operands' bytes are widened
// to bf16, exactly, on their way to LDS and contracted by v_mfma_f32_32x32x16_bf16.  Measured on gfx950: that
// instruction keeps every product bit down to 2^-24 of the largest term of its 16-long k block and rounds the
// block sum plus accumulator to nearest even, so a contraction stays within the error bound of a float32
// summation; the fp8 MFMA forms (v_mfma_f32_32x32x16_fp8_fp8 and v_mfma_scale_f32_32x32x64_f8f6f4 alike) align
// the products of every 8 consecutive k to the largest of them and cut each off 2^-13 below it.  Half the
// matrix-core rate and twice the LDS bytes of the fp8 form.
template <int FMT_A, int FMT_B>
struct MmaBf16F8 {
  typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
  using Acc = v16f;
  using AccScalar = float;
  using Frag = v4i;
  static constexpr int kChunks = 1;
  static constexpr bool kIntAcc = false;
  static constexpr bool kWidenA = true, kWidenB = true;
  static __device__ __forceinline__ Acc mma(const Frag& x, const Frag& y, const Acc& c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, x), __builtin_bit_cast(v8bf, y), c, 0, 0, 0);
  }
  static __device__ __forceinline__ void widen_a(const v4i x4, v4i& lo, v4i& hi) { widen_f8x16_bf16<FMT_A>(x4, lo, hi); }
  static __device__ __forceinline__ void widen_b(const v4i x4, v4i& lo, v4i& hi) { widen_f8x16_bf16<FMT_B>(x4, lo, hi); }
};

struct GemmArgs {
  const uint8_t* a;
  const uint8_t* b;
  const float* row_scale;
  const float* col_scale;
  void* c;
  void* acc_out;   // int32 (int8 operands) or float (fp8 operands)
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t stride_a, stride_b, stride_c, stride_rs, stride_cs;
  int tiles_m, tiles_n;
  int out_dtype;  // AQTX_BF16 | AQTX_F32 | AQTX_I32
  int dq_bf16;    // dequant dtype is bf16
  int p1_bf16;    // the first product is rounded to bf16
  int p2_bf16;    // the second product is rounded to bf16
  int col_first;  // scale order
  // Ragged batches: entry b multiplies rows [group_offsets[b], group_offsets[b+1]) of one flat
  // A with B[b] into the same rows of one flat C (m is then an upper bound of a group's rows).
  const int32_t* group_offsets;
  int a_even_odd8;  // packed int4 B only: A's bytes of every 8 k are stored as k 0,2,4,6,1,3,5,7
  // B in the fragment order of aqtx_tile_weight (batch 1): blocks of 16 rows, b_steps KiB each, a KiB holding
  // 64 bytes of each of the 16 rows (lane r + 16 c of the KiB = bytes 16 c .. 16 c + 15 of row r); rows past n
  // and bytes past the row's end are zeros there.
  int b_frag, b_steps;
  // Split K (gemm_mid_kernel): workgroup z of the grid contracts k in [z * k_chunk, (z + 1) * k_chunk) and
  // writes its int32 partial sums to slab z of `slabs` ([k_split][batch][m][n]); dequant_slabs_kernel adds
  // the slabs (integer addition: exact) and dequantizes.
  int k_split;      // slices (<= 1: none)
  int64_t k_chunk;  // k per slice, a multiple of 128
  int32_t* slabs;
  // Convolution (gemm_mid_kernel<..., CONV>): A is not a matrix but the int8 input [images][spatial...][c]; row
  // r of the contraction is output position r, k runs over the kernel window in tap order with the features
  // innermost, and what lies in the padding reads as zero.  Up to three spatial axes, missing leading ones 1.
  struct {
    int32_t c;
    int32_t in[3], ker[3], str[3], dil[3], pad[3], osz[3];
    int64_t x_bytes;
  } conv;
};

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kTileBytes = BM * BK;          // one operand tile of one stage: 32 KiB
constexpr int kStageBytes = 2 * kTileBytes;  // A tile + B tile
constexpr uint32_t kBufferRsrcWord3 = 0x00020000u;  // raw buffer, 32-bit data format (gfx9)

#define AQTX_LDS_PTR(p) ((__attribute__((address_space(3))) void*)(p))

__device__ __forceinline__ float rnd(float x, int bf) { return bf ? round_bf16(x) : x; }

// 16 bytes of packed int4 (32 values, low nibble = even k) -> 32 bytes of values * 16 in k order.
// dword d of the load = k 8d..8d+7: even k: (x << 4) & 0xF0F0F0F0, odd k: x & 0xF0F0F0F0; then
// the bytes are interleaved back to k order.
// With even_odd8 the other operand stores every 8 k as k 0,2,4,6,1,3,5,7, and the interleaving is left out.
__device__ __forceinline__ void unpack_i4x32(const v4i x4, v4i& lo, v4i& hi, int even_odd8) {
  if (even_odd8) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t x = (uint32_t)x4[d];
      const int ev = (int)((x << 4) & 0xF0F0F0F0u), od = (int)(x & 0xF0F0F0F0u);
      if (d < 2) { lo[2 * d] = ev; lo[2 * d + 1] = od; }
      else { hi[2 * (d - 2)] = ev; hi[2 * (d - 2) + 1] = od; }
    }
    return;
  }
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const uint32_t x = (uint32_t)x4[d];
    const uint32_t ev = (x << 4) & 0xF0F0F0F0u, od = x & 0xF0F0F0F0u;
    const uint32_t k03 = __builtin_amdgcn_perm(od, ev, 0x05010400u);  // e0 o0 e1 o1
    const uint32_t k47 = __builtin_amdgcn_perm(od, ev, 0x07030602u);  // e2 o2 e3 o3
    if (d < 2) { lo[2 * d] = (int)k03; lo[2 * d + 1] = (int)k47; }
    else { hi[2 * (d - 2)] = (int)k03; hi[2 * (d - 2) + 1] = (int)k47; }
  }
}


// Workgroup id -> tile, XCD-aware: ids are dealt round-robin to the 8 XCDs, so id%8
// picks the XCD; each XCD then walks a contiguous range of tiles in bands of 8 tile
// rows, keeping the operand panels of concurrently running tiles in its own L2.
__device__ __forceinline__ void tile_of_block(int bid, int tiles_m, int tiles_n, int& tm, int& tn) {
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + 7) / 8;
  int id = (bid % 8) * per_xcd + bid / 8;
  if (total % 8 != 0) id = bid;  // uneven split: keep the plain order
  constexpr int kBand = 8;
  const int band_tiles = kBand * tiles_n;
  const int band = id / band_tiles;
  const int first_m = band * kBand;
  const int rows_in_band = (tiles_m - first_m) < kBand ? (tiles_m - first_m) : kBand;
  const int in_band = id % band_tiles;
  tm = first_m + in_band % rows_in_band;
  tn = in_band / rows_in_band;
}

// QTensor.dequant of one accumulator for epilogue EPI (see gemm_kernel): cast to the dequant dtype, times
// the first scale, times the second, each product rounded to the promoted dtype of its operands.
template <int EPI, bool COL_FIRST, class AccScalar>
__device__ __forceinline__ float dequant_value(AccScalar accv, float s_row, float s_col) {
  constexpr bool kDqBf16 = EPI <= 1 || EPI == 4;
  constexpr bool kProd1Bf16 = EPI == 0 || EPI == 4;     // promote(dequant dtype, first scale dtype)
  constexpr bool kProd2Bf16 = EPI == 0;                 // promote(that, second scale dtype)
  float f = round_to<kDqBf16>((float)accv);  // (int32 ->) f32 -> dequant dtype
  const float s1 = COL_FIRST ? s_col : s_row, s2 = COL_FIRST ? s_row : s_col;
  f = round_to<kProd1Bf16>(f * s1);
  f = round_to<kProd2Bf16>(f * s2);
  return round_to<kDqBf16>(f);
}

// EPI selects the epilogue arithmetic at compile time (run-time flags there turn into
// thousands of branches): 0 = bf16 out, bf16 scales; 1 = bf16 out, first scale f32; 2 = f32 out;
// 3 = raw accumulators only; 4 = bf16 out, first scale bf16, second f32.  COL_FIRST: the column scale multiplies first.
// KTAIL: K is not a multiple of the 128-byte stage, the last stage masks chunks past K.
// NW: waves per workgroup.  4 = 2x2 waves with 128x128 wave tiles, one wave per SIMD;
// 8 = 2x4 waves with 128x64 wave tiles, two waves per SIMD, so that one wave's MFMAs fill the
// issue slots in which the other waits on the memory pipeline.
// BPACK (int8 MFMA only): B holds int4 values packed two per byte ([n][k/2], low nibble = even k; ldb and
// stride_b in bytes).  A wave load then covers 16 rows x 64 B, and a lane's 16 bytes are unpacked in
// registers into the two neighbouring 16-byte chunks of its row on their way to LDS: a nibble is
// moved to the top of its byte (value * 16); the epilogue takes the factor 16 out again, exactly (a
// power of two commutes with every rounding of the dequantisation).
// PERSIST: the grid has one workgroup per CU (or fewer) and a workgroup walks tiles blockIdx.x, + gridDim.x, ...
// (the XCD-aware order of tile_of_block continues: a workgroup stays on its XCD's range).  Between two tiles no
// workgroup has to be launched, and the first stage of the next tile is requested before the epilogue of this one
// (packed operands: the staging registers are free then), so its latency passes under the stores.  Plain batches only.
template <class MMA, int NW, int EPI, bool COL_FIRST, bool KTAIL, bool BPACK = false, bool BFRAG = false, bool PERSIST = false>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW / 4, NW / 4)))
void gemm_kernel(const GemmArgs g_in) {
  static_assert(NW == 4 || NW == 8, "4 or 8 waves");
  static_assert(!BFRAG || MMA::kIntAcc || MMA::kWidenB, "the fragment order is that of int8 / packed int4 weights");
  static_assert(!BPACK || MMA::kIntAcc || MMA::kWidenB, "packed int4 goes with the int8 MFMA, int8 to widen with a bf16 one");
  static_assert(BPACK || !MMA::kWidenB, "a B that is widened on its way to LDS takes the packed loads");
  // the nibbles of a packed int4 B sit at the top of their bytes: the accumulators hold 16 times the contraction
  constexpr bool kTimes16 = BPACK && MMA::kIntAcc;
  GemmArgs g = g_in;
  constexpr int NI = 16 / NW;       // 32-column MFMA tiles per wave
  constexpr int WN = NW / 2;        // waves along n
  constexpr int LPW = 32 / NW;      // 8-row load blocks per wave and operand
  constexpr int NL = 2 * LPW;       // LDS stores per wave and stage
  constexpr int LPB = BPACK ? LPW / 2 : LPW;  // B loads per wave and stage
  constexpr int NLD = LPW + LPB;    // global loads per wave and stage
  constexpr int MPK = 4 * NI;       // MFMAs per wave and k-step
  using Acc = typename MMA::Acc;
  using AccScalar = typename MMA::AccScalar;
  using Frag = typename MMA::Frag;
  constexpr int kChunks = MMA::kChunks;
  constexpr int KS = 4 / kChunks;  // k-steps (rounds of MPK MFMAs) per 128-byte stage
  // Two stages in two distinct LDS objects, so that the compiler can tell the stage
  // being filled by the buffer->LDS loads from the one the MFMA fragments are read from.
  __shared__ __attribute__((aligned(1024))) uint8_t stage0[kStageBytes];
  __shared__ __attribute__((aligned(1024))) uint8_t stage1[kStageBytes];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lr = lane & 31, lh = lane >> 5;

  int tm, tn;
  if (g_in.group_offsets != nullptr) {
    // Only the first few tile rows of a group hold work; ids run along n first, so that those
    // rows are dealt round-robin to all XCDs (the banded walk would leave them to one XCD).
    tm = (int)(blockIdx.x / (unsigned)g.tiles_n);
    tn = (int)(blockIdx.x % (unsigned)g.tiles_n);
  } else {
    tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  }
  const int64_t bz = blockIdx.y;
  int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  if (g_in.group_offsets != nullptr) {
    // the group's row range replaces the batch strides of A, C and the row scale; tiles past
    // the group's last row leave at once (the grid is sized for the largest possible group)
    const int64_t row0 = g_in.group_offsets[bz];
    const int64_t rows = g_in.group_offsets[bz + 1] - row0;
    if (m0 >= rows) return;
    g.m = rows;
    g.a += row0 * g.lda;
    g.c = reinterpret_cast<uint8_t*>(g.c) + row0 * g.ldc * (g.out_dtype == AQTX_BF16 ? 2 : 4);
    if (g.acc_out != nullptr) g.acc_out = reinterpret_cast<uint8_t*>(g.acc_out) + row0 * g.ldc * 4;
    if (g.row_scale != nullptr) g.row_scale += row0;
    g.stride_a = 0; g.stride_c = 0; g.stride_rs = 0;
  }

  // ---- global -> LDS.  One wave instruction moves 8 rows x 128 B (1 KiB): lane l handles LDS slot
  // (row l>>3, chunk l&7) of its 8-row block and fetches the global chunk (l&7) ^ f(row),
  // f(row) = (row ^ row>>3) & 7, which is the XOR swizzle the fragment reads undo.  Rows past the end of
  // the operand fall outside the buffer and read as zero.  A stage buffer is only free for refilling at the
  // end of a stage (behind the barrier that stands before the last k step).  Unpacked operands are requested
  // there straight into it (buffer load to LDS, one request per matrix instruction of that k step; the same
  // 64 KiB requested in one burst right behind the barrier queued up in the CU's address unit while the waves
  // that issued them could not issue MFMAs).  Packed operands, and the first stage of a tile, go through
  // registers: requested a few MFMAs apart over the stage, written to the freed buffer with ds_write.
  // BFRAG, B in fragment order (GemmArgs::b_frag): the tile's 16-row blocks follow one another, b_steps KiB
  // each; the piece (row r, 16 bytes at 16 c of a 64-byte step) is lane r % 16 + 16 c of its KiB, and the scalar
  // offset of a stage is its row bytes times 16.
  auto rsrc_a_of = [&](int64_t tm0) {
    const int64_t rows_a = (g.m - tm0) < BM ? (g.m - tm0) : BM;
    return __builtin_amdgcn_make_buffer_rsrc((void*)(g.a + bz * g.stride_a + tm0 * g.lda), 0,
                                             (int)((rows_a - 1) * g.lda + g.k), kBufferRsrcWord3);
  };
  auto rsrc_b_of = [&](int64_t tn0) {
    const int64_t rows_b = (g.n - tn0) < BN ? (g.n - tn0) : BN;
    return BFRAG ? __builtin_amdgcn_make_buffer_rsrc((void*)(g.b + (tn0 / 16) * (int64_t)g.b_steps * 1024), 0,
                                                     (int)((rows_b + 15) / 16 * g.b_steps * 1024), kBufferRsrcWord3)
                 : __builtin_amdgcn_make_buffer_rsrc((void*)(g.b + bz * g.stride_b + tn0 * g.ldb), 0,
                                                     (int)((rows_b - 1) * g.ldb + (BPACK ? g.k / 2 : g.k)), kBufferRsrcWord3);
  };
  __amdgpu_buffer_rsrc_t rsrc_a = rsrc_a_of(m0), rsrc_b = rsrc_b_of(n0);
  constexpr int ksh_b = BFRAG ? 4 : 0;
  // Unpacked B in fragment order keeps that order in LDS: KiB blk of the B tile's stage is half blk & 1 of 16-row
  // block blk >> 1, as it lies in memory, so that a wave's request is one contiguous KiB (asking for the pieces
  // the swizzled row layout wants, 16 bytes from each of 64 places of two KiB, cost 146 against 129 us on
  // 2048 x 4096 x 14336).
  constexpr bool kFragLds = BFRAG && !BPACK;
  static_assert(!kFragLds || MMA::kChunks == 1, "fragment order: 16 bytes of a row per lane and k step");
  int voff_a[LPW], voff_b[LPB], chunk_byte[LPW];
#pragma unroll
  for (int i = 0; i < LPW; ++i) {
    const int blk = wave * LPW + i;
    const int row = blk * 8 + (lane >> 3);
    chunk_byte[i] = (((lane & 7) ^ (lane >> 3) ^ blk) & 7) * 16;
    voff_a[i] = row * (int)g.lda + chunk_byte[i];
    if constexpr (kFragLds) voff_b[i] = ((blk >> 1) * g.b_steps + (blk & 1)) * 1024 + lane * 16;
    else if constexpr (!BPACK) voff_b[i] = row * (int)g.ldb + chunk_byte[i];
  }
  // position along k of lane's 16 bytes of B piece i (for the mask on K)
  auto kpos_b = [&](int i) -> int { return kFragLds ? ((wave * LPW + i) & 1) * 64 + (lane >> 4) * 16 : chunk_byte[i]; };
  // packed B: load q of a wave covers rows 16 (wave LPB + q) .. +15, lane -> row lane >> 2, 16 packed bytes
  // (32 k) at 16 (lane & 3); they become the chunks 2p, 2p + 1 of that row, at positions chunk ^ f(row)
  int pb_st[LPB];
  if constexpr (BPACK) {
#pragma unroll
    for (int q = 0; q < LPB; ++q) {
      const int row = (wave * LPB + q) * 16 + (lane >> 2);
      voff_b[q] = BFRAG ? (wave * LPB + q) * g.b_steps * 1024 + ((lane & 3) * 16 + (lane >> 2)) * 16
                        : row * (int)g.ldb + (lane & 3) * 16;
      pb_st[q] = kTileBytes + row * BK + (((2 * (lane & 3)) ^ ((row ^ (row >> 3)) & 7)) * 16);
    }
  }
  // Loads and stores are numbered in the order they are issued.  Unpacked: A block i, B block i alternate
  // (load j = store j).  Packed: A0 B0 A1 | A2 B1 A3 | ..., and a B load feeds two stores.
  v4i stga[LPW], stgb[LPB], pb_hi[LPB];
  auto load_global = [&](int j, int k0) {  // j = 0..NLD-1
    const bool is_b = BPACK ? (j % 3 == 1) : (j & 1);
    const int i = BPACK ? (is_b ? j / 3 : j - (j + 1) / 3) : (j >> 1);
    if (!is_b) {
      int vo = voff_a[i];
      if (KTAIL && k0 + chunk_byte[i] >= (int)g.k) vo = 0x7FFFFFF0;  // out of range -> zeros
      stga[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, vo, k0, 0);
    } else if constexpr (BPACK) {
      int vo = voff_b[i];
      if (KTAIL && k0 + (lane & 3) * 32 >= (int)g.k) vo = 0x7FFFFFF0;
      stgb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, (k0 / 2) << ksh_b, 0);
    } else {
      int vo = voff_b[i];
      if (KTAIL && k0 + kpos_b(i) >= (int)g.k) vo = 0x7FFFFFF0;
      stgb[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo, k0 << ksh_b, 0);
    }
  };
  const int st_off = wave * LPW * 1024 + lane * 16;
  // Unpacked operands refill a stage buffer straight from memory (buffer load to LDS: lane i's 16 bytes land at
  // base + 16 i, which is the layout above), one request per matrix instruction of the stage's last k step,
  // with no ds_write: a stage's 64 ds_write_b128 (8 cycles each) added their 470 cycles to the 2070 the stage
  // takes without them, wherever in the stage they stood (clock stamps: 2550 cycles a stage through registers,
  // 2220-2300 this way).  Packed operands are unpacked in registers and keep that path.
  constexpr bool kDirect = !BPACK;
  auto load_direct = [&](uint8_t* st, int j, int k0) {  // piece j (the numbering of load_global) of the stage at k0
    const bool is_b = j & 1;
    const int i = j >> 1;
    int vo = is_b ? voff_b[i] : voff_a[i];
    if (KTAIL && k0 + (is_b ? kpos_b(i) : chunk_byte[i]) >= (int)g.k) vo = 0x7FFFFFF0;  // out of range -> zeros
    uint8_t* at = st + (is_b ? kTileBytes : 0) + wave * LPW * 1024 + i * 1024;  // wave-uniform
    if (!is_b) __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)at, 16, vo, k0, 0, 0);
    else __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_b, (__attribute__((address_space(3))) void*)at, 16, vo, k0 << ksh_b, 0, 0);
  };
  auto store_lds = [&](uint8_t* st, int j) {  // j = 0..NL-1
    if constexpr (!BPACK) {
      const int i = j >> 1;
      *reinterpret_cast<v4i*>(st + ((j & 1) ? kTileBytes : 0) + st_off + i * 1024) = (j & 1) ? stgb[i] : stga[i];
    } else {
      // stores in the order of the loads: A0 B0.lo B0.hi A1 | A2 B1.lo B1.hi A3 | ...
      const int grp = j >> 2, r4 = j & 3;
      if (r4 == 0 || r4 == 3) {
        const int i = 2 * grp + (r4 == 3 ? 1 : 0);
        *reinterpret_cast<v4i*>(st + st_off + i * 1024) = stga[i];
      } else if (r4 == 1) {
        v4i lo;
        if constexpr (MMA::kWidenB) MMA::widen_b(stgb[grp], lo, pb_hi[grp]);
        else unpack_i4x32(stgb[grp], lo, pb_hi[grp], g.a_even_odd8);
        *reinterpret_cast<v4i*>(st + pb_st[grp]) = lo;
      } else {
        *reinterpret_cast<v4i*>(st + (pb_st[grp] ^ 16)) = pb_hi[grp];
      }
    }
  };

  // ---- per-lane swizzled fragment offsets: chunk ((2*ks + lh) * kChunks + c) ^ f(row)
  const int lf0 = (lr ^ (lr >> 3)) & 7;
  int frag_off[8];
#pragma unroll
  for (int cidx = 0; cidx < 8; ++cidx)
    frag_off[cidx] = lr * BK + (((lh * kChunks) ^ lf0 ^ cidx) * 16);
  // B kept in fragment order: chunk q = 2 ks + lh of row r of a 32-row block lies at
  // (2 (r >> 4) + (q >> 2)) KiB + 16 (16 (q & 3) + (r & 15)); the 16 rows of a read are consecutive
  int frag_off_b[4];
#pragma unroll
  for (int ks = 0; ks < 4; ++ks) {
    const int q = 2 * ks + lh;
    frag_off_b[ks] = (2 * (lr >> 4) + (q >> 2)) * 1024 + (16 * (q & 3) + (lr & 15)) * 16;
  }
  const int a_base = wm * 128 * BK;                // rows of the A tile this wave needs
  const int b_base = kTileBytes + wn * NI * 32 * BK;   // rows of the B tile

  Acc acc[4][NI];

  auto load_frag = [&](const uint8_t* rows, int ks, int i) -> Frag {
    if constexpr (kChunks == 1) {
      return *reinterpret_cast<const v4i*>(rows + i * 32 * BK + frag_off[(2 * ks) ^ (4 * (i & 1))]);
    } else {
      const int c0 = (4 * ks) ^ (4 * (i & 1)), c1 = c0 ^ 1;
      const v4i x0 = *reinterpret_cast<const v4i*>(rows + i * 32 * BK + frag_off[c0]);
      const v4i x1 = *reinterpret_cast<const v4i*>(rows + i * 32 * BK + frag_off[c1]);
      return Frag{x0[0], x0[1], x0[2], x0[3], x1[0], x1[1], x1[2], x1[3]};
    }
  };
  auto load_frags = [&](const uint8_t* st, int ks, Frag* fa, Frag* fb) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      fa[i] = load_frag(st + a_base, ks, i);
      if constexpr (kFragLds) {
        if (i < NI) fb[i] = *reinterpret_cast<const v4i*>(st + b_base + i * 32 * BK + frag_off_b[ks]);
      } else {
        if (i < NI) fb[i] = load_frag(st + b_base, ks, i);
      }
    }
  };
  auto mfma_step = [&](const Frag* fa, const Frag* fb) {
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni) acc[mi][ni] = MMA::mma(fb[ni], fa[mi], acc[mi][ni]);
  };
  // Scheduling groups (llvm.amdgcn.sched.group.barrier masks).
  constexpr int kMfma = 0x008, kVmemRead = 0x020, kDsRead = 0x100, kDsWrite = 0x200;

  // Software pipeline of one stage (KS k-steps of 16 MFMAs):
  //   k-steps 0..KS-2: fragments of the next k-step are read from LDS (spread over the MFMAs);
  //                 packed operands: the global loads of the block two stages ahead are issued a few
  //                 MFMAs apart, into the staging registers;
  //   barrier     : every wave holds its last fragments of this stage, the buffer is free; with direct
  //                 refills each wave has first waited for its own requests into the other buffer;
  //   last k-step : the freed buffer is refilled with the block two stages ahead, one request (direct) or
  //                 one ds_write from the staging registers (packed, each waiting only for its own load)
  //                 per MFMA, and the first fragments of the next stage are read from the other buffer.
  // The barrier is a bare s_barrier: a __syncthreads() would also wait for the global loads
  // still in flight.  No branch surrounds any MFMA (a conditional stage makes the compiler
  // shuffle all 256 accumulators through VGPRs).
  Frag fa0[4], fb0[NI], fa1[4], fb1[NI];
  constexpr int kDsPerStep = (4 + NI) * kChunks;  // ds_read_b128 per k-step
  auto run_stage = [&](const uint8_t* cur, uint8_t* cur_refill, const uint8_t* next, int refill_k0) {
#pragma unroll
    for (int ks = 0; ks < KS - 1; ++ks) {
      // loads [l0, l1) of the 16 go with this k-step
      const int l0 = (NLD * ks + KS - 2) / (KS - 1), l1 = (NLD * (ks + 1) + KS - 2) / (KS - 1);
      if (ks % 2 == 0) load_frags(cur, ks + 1, fa1, fb1); else load_frags(cur, ks + 1, fa0, fb0);
      if constexpr (!kDirect) {
#pragma unroll
        for (int j = l0; j < l1; ++j) load_global(j, refill_k0);
      }
      if (ks % 2 == 0) mfma_step(fa0, fb0); else mfma_step(fa1, fb1);
      const int nl = kDirect ? 0 : l1 - l0;
#pragma unroll
      for (int i = 0; i < MPK; ++i) {
        __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
        if (i < kDsPerStep) __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
        const bool slot = (MPK == 16 && nl == 6) ? (i % 3 == 0)
                        : (MPK == 16 && nl == 5) ? (i % 3 == 1)
                        : ((i + 1) * nl / MPK > i * nl / MPK);
        if (slot) __builtin_amdgcn_sched_group_barrier(kVmemRead, 1, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    // direct refills: this wave's pieces of the other buffer (requested a stage ago) have landed, and after the
    // barrier so have everybody's
    if constexpr (kDirect) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kDirect) {
#pragma unroll
      for (int j = 0; j < NL; ++j) load_direct(cur_refill, j, refill_k0);
    } else {
#pragma unroll
      for (int j = 0; j < NL; ++j) store_lds(cur_refill, j);
    }
    // KS is even, so the last k-step always computes from set 1 and refills set 0.
    load_frags(next, 0, fa0, fb0);
    mfma_step(fa1, fb1);
#pragma unroll
    for (int i = 0; i < MPK; ++i) {
      __builtin_amdgcn_sched_group_barrier(kMfma, 1, 0);
      if (kDirect) __builtin_amdgcn_sched_group_barrier(kVmemRead, 1, 0);
      else __builtin_amdgcn_sched_group_barrier(kDsWrite, 1, 0);
      if (i < kDsPerStep) __builtin_amdgcn_sched_group_barrier(kDsRead, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // An odd number of 128-byte K blocks is rounded up: with KTAIL the extra block is masked
  // to zeros; without it K is a multiple of 256 bytes and no extra block exists.
  const int KT2 = (int)((g.k + 2 * BK - 1) / (2 * BK));
  // The scalar offset of a buffer load is not part of the hardware's range check, so a block
  // requested past the end of K would really be fetched (up to 256 bytes past the last row of
  // the operand).  Without KTAIL the two look-ahead requests of the last trip are redirected to
  // the last block of K instead (a scalar minimum; their data is never consumed); with KTAIL
  // the per-chunk mask in load_global already covers them.
  const int k0_last = KTAIL ? 0x7FFFFF00 : (int)g.k - BK;
  auto refill_at = [&](int k0) { return k0 < k0_last ? k0 : k0_last; };
  if constexpr (!kDirect) {
#pragma unroll
    for (int j = 0; j < NLD; ++j) load_global(j, 0);
  }
  int tile = (int)blockIdx.x;
  for (;;) {  // one trip per tile (one trip unless PERSIST)
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < NI; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
  if constexpr (kDirect) {
    // (both stages straight into LDS: asking for the first one before the previous tile's epilogue, into
    // registers, saved a thousand cycles a tile and cost ten spilled registers; measured level or 1 % behind.
    // Asking for both straight into LDS before the epilogue, which then passed its rows 32 at a time through
    // 32 KiB of its own: level on all-zero operands, 1 % behind on N(0, 25) ones, 6-10 spilled registers)
#pragma unroll
    for (int j = 0; j < NL; ++j) load_direct(stage0, j, 0);
#pragma unroll
    for (int j = 0; j < NL; ++j) load_direct(stage1, j, BK);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
#pragma unroll
    for (int j = 0; j < NL; ++j) store_lds(stage0, j);
#pragma unroll
    for (int j = 0; j < NLD; ++j) load_global(j, BK);
#pragma unroll
    for (int j = 0; j < NL; ++j) store_lds(stage1, j);
  }
  __syncthreads();
  load_frags(stage0, 0, fa0, fb0);
  for (int it = 0; it < KT2; ++it) {
    run_stage(stage0, stage0, stage1, refill_at((2 * it + 2) * BK));
    run_stage(stage1, stage1, stage0, refill_at((2 * it + 3) * BK));
  }
  // (direct refills requested past the end of k re-read its last block: they have to land before the epilogue
  // stages the output in the same buffers)
  if constexpr (kDirect) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // ---- epilogue ---------------------------------------------------------------
  // lane holds C[m = mrow0 + mi*32 + lr][n = ncol0 + ni*32 + 8*q + 4*lh + e], e = 0..3, reg = 4*q+e
  const int64_t em0 = m0, en0 = n0;  // this tile's corner: m0, n0 move on to the next tile below
  const int64_t mrow0 = em0 + wm * 128, ncol0 = en0 + wn * NI * 32;
  bool more = false;
  if constexpr (PERSIST) {
    // packed operands: the next tile's first stage is requested now: the staging registers are free, and the
    // epilogue's stores hide the latency
    tile += (int)gridDim.x;
    more = tile < g.tiles_m * g.tiles_n;
    if (more) {
      tile_of_block(tile, g.tiles_m, g.tiles_n, tm, tn);
      m0 = (int64_t)tm * BM; n0 = (int64_t)tn * BN;
      rsrc_a = rsrc_a_of(m0); rsrc_b = rsrc_b_of(n0);
      if constexpr (!kDirect) {
#pragma unroll
        for (int j = 0; j < NLD; ++j) load_global(j, 0);
      }
    }
  }

  if (g.acc_out != nullptr) {  // optional second copy of the raw accumulators (plain stores)
    AccScalar* dst = reinterpret_cast<AccScalar*>(g.acc_out);
    dst += bz * g.stride_c;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t mm = mrow0 + mi * 32 + lr;
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t nn = ncol0 + ni * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (mm < g.m && nn < g.n) {
            if constexpr (kTimes16) dst[mm * g.ldc + nn] = acc[mi][ni][r] >> 4;  // exact: a multiple of 16
            else dst[mm * g.ldc + nn] = acc[mi][ni][r];
          }
        }
    }
  }
  {
    // EPI 3 (raw accumulators as the output) takes the same staged, coalesced store path as the
    // float outputs: the 32-bit patterns travel through the float slots untouched.
    constexpr bool kOutBf16 = EPI <= 1 || EPI == 4;       // dequant dtype == output dtype
    // A missing scale is a multiplication by 1, which every rounding below leaves alone.
    const float* rs = g.row_scale ? g.row_scale + bz * g.stride_rs : nullptr;
    const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
    float rscale[4];
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t mm = mrow0 + mi * 32 + lr;
      rscale[mi] = (rs != nullptr && mm < g.m) ? rs[mm] : 1.0f;
    }
    auto dequant = [&](AccScalar accv, float s_row, float s_col) {
      if constexpr (EPI == 3) {
        if constexpr (kTimes16) return __builtin_bit_cast(float, accv >> 4);
        else return __builtin_bit_cast(float, accv);
      }
      return dequant_value<EPI, COL_FIRST>(accv, s_row, s_col);
    };

    // Each wave stages its 128-row block in LDS, RB = 256 (4 waves) or 128 (8 waves) bytes per
    // row, no padding: the 8-byte chunk j of row r sits at chunk j ^ sw(r), sw chosen so that
    // the 32 lanes that write one column group hit 32 distinct bank pairs, and a row is read
    // back as aligned 16-byte pairs.
    //   bf16: one pass over the NI n-tiles; f32: two passes of NI/2 n-tiles (same row bytes).
    constexpr int kPasses = kOutBf16 ? 1 : 2;
    constexpr int kNiPerPass = kOutBf16 ? NI : NI / 2;
    constexpr int kEsz = kOutBf16 ? 2 : 4;
    constexpr int RB = kNiPerPass * 32 * kEsz;
    static_assert(RB == NI * 64, "row bytes");
    constexpr int kColsPerPair = 16 / kEsz;
    uint8_t* region = (wave < NW / 2 ? stage0 : stage1) + (wave % (NW / 2)) * (128 * RB);
    auto sw_of = [](int row) { return RB == 256 ? (row & 31) : ((row >> 1) & 15); };
    uint8_t* cbase = reinterpret_cast<uint8_t*>(g.c) + bz * g.stride_c * kEsz;
    const bool vec_store = ((g.ldc * kEsz) % 16) == 0 && ((uintptr_t)cbase % 16) == 0;
    // Tiles that lie wholly inside C and can use 16-byte stores skip every bounds check.
    const bool interior = vec_store && (em0 + BM <= g.m) && (en0 + BN <= g.n);

    auto epilogue = [&](auto checked_tag) {
      constexpr bool kChecked = decltype(checked_tag)::value;
#pragma unroll
      for (int pass = 0; pass < kPasses; ++pass) {
#pragma unroll
        for (int nj = 0; nj < kNiPerPass; ++nj) {
          const int ni = pass * kNiPerPass + nj;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int ncol_local = nj * 32 + 8 * q + 4 * lh;  // within the pass
            const int64_t nn = ncol0 + ni * 32 + 8 * q + 4 * lh;
            float csv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
            if (cs != nullptr) {
              if constexpr (kChecked) {
#pragma unroll
                for (int e = 0; e < 4; ++e) csv[e] = (nn + e < g.n) ? cs[nn + e] : 1.0f;
              } else {
                const float4 c4 = *reinterpret_cast<const float4*>(cs + nn);
                csv[0] = c4.x; csv[1] = c4.y; csv[2] = c4.z; csv[3] = c4.w;
              }
            }
            if constexpr (kTimes16) {  // the accumulators hold 16 times the contraction
#pragma unroll
              for (int e = 0; e < 4; ++e) csv[e] *= 0.0625f;
            }
#pragma unroll
            for (int mi = 0; mi < 4; ++mi) {
              float o[4];
#pragma unroll
              for (int e = 0; e < 4; ++e) o[e] = dequant(acc[mi][ni][4 * q + e], rscale[mi], csv[e]);
              const int row = mi * 32 + lr;
              uint8_t* p = region + row * RB;
              const int sw = sw_of(row);
              if constexpr (kOutBf16) {
                uint2 w;
                w.x = (uint32_t)bf16_bits(o[0]) | ((uint32_t)bf16_bits(o[1]) << 16);
                w.y = (uint32_t)bf16_bits(o[2]) | ((uint32_t)bf16_bits(o[3]) << 16);
                const int j = ncol_local >> 2;  // 8-byte chunk index
                *reinterpret_cast<uint2*>(p + ((j ^ sw) * 8)) = w;
              } else {
                const int j = ncol_local >> 1;  // two 8-byte chunks per 4 floats
                *reinterpret_cast<float2*>(p + ((j ^ sw) * 8)) = make_float2(o[0], o[1]);
                *reinterpret_cast<float2*>(p + (((j + 1) ^ sw) * 8)) = make_float2(o[2], o[3]);
              }
            }
          }
        }
        // (no barrier: the region is this wave's own, and a wave's LDS accesses complete in order)
        // read back: lane -> 16-byte pair (lane % LPR) of row (lane / LPR) + RPI*it
        constexpr int LPR = RB / 16, RPI = 64 / LPR;
        const int64_t ncol_pass0 = ncol0 + (int64_t)pass * kNiPerPass * 32;
        const int pair = lane % LPR, rsub = lane / LPR;
        const int64_t nn = ncol_pass0 + pair * kColsPerPair;
        const bool full = vec_store && (nn + kColsPerPair <= g.n);
        uint8_t* dst0 = cbase + ((mrow0 + rsub) * g.ldc + nn) * kEsz;
#pragma unroll 8
        for (int it = 0; it < 128 / RPI; ++it) {
          const int row = rsub + RPI * it;
          const int sw = sw_of(row);
          uint4 v = *reinterpret_cast<const uint4*>(region + row * RB + ((pair ^ (sw >> 1)) * 16));
          if (sw & 1) v = make_uint4(v.z, v.w, v.x, v.y);
          uint8_t* dst = dst0 + (int64_t)it * RPI * g.ldc * kEsz;
          // Non-temporal: the output is not read again by this launch, and kept out of the L2 it leaves the
          // operand panels there (measured: 0.7 % off the launch, 1.4 % off the training step)
          const v4i vo = v4i{(int)v.x, (int)v.y, (int)v.z, (int)v.w};
          if constexpr (!kChecked) {
            __builtin_nontemporal_store(vo, reinterpret_cast<v4i*>(dst));
          } else if (mrow0 + row < g.m && nn < g.n) {
            if (full) {
              __builtin_nontemporal_store(vo, reinterpret_cast<v4i*>(dst));
            } else {
              const uint32_t w[4] = {v.x, v.y, v.z, v.w};
              const int nv = (int)(g.n - nn) < kColsPerPair ? (int)(g.n - nn) : kColsPerPair;
              for (int e = 0; e < nv; ++e) {
                if constexpr (kOutBf16)
                  reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
                else
                  reinterpret_cast<uint32_t*>(dst)[e] = w[e];
              }
            }
          }
        }
      }
    };
    if (interior && ((uintptr_t)cs % 16) == 0) epilogue(std::false_type{});
    else epilogue(std::true_type{});
  }
  if (!more) break;
  __syncthreads();  // the staging rows of the epilogue have been read: the next tile may fill the stages
  }
}

// Second step of a split-K contraction: C = dequant(sum of the k_split int32 slabs [batch][m][n]) with the
// arithmetic of the fused epilogue EPI (0, 1, 2, 4; 3 = the raw sums); also writes the sums to acc_out when
// that is given.  One thread per four neighbouring columns.
template <int EPI, bool COL_FIRST>
__global__ __launch_bounds__(256) void dequant_slabs_kernel(const GemmArgs g) {
  constexpr bool kOutBf16 = EPI <= 1 || EPI == 4;
  const int64_t n4 = (int64_t)(blockIdx.x * 256 + threadIdx.x) * 4;
  const int64_t mm = blockIdx.y, bz = blockIdx.z;
  if (n4 >= g.n) return;
  const int nv = (g.n - n4) < 4 ? (int)(g.n - n4) : 4;
  const int64_t slab = (int64_t)gridDim.z * g.m * g.n;
  const int64_t so = (bz * g.m + mm) * g.n + n4;
  int a4[4] = {0, 0, 0, 0};
  const bool svec = nv == 4 && (g.n % 4) == 0;
  for (int z = 0; z < g.k_split; ++z) {
    const int32_t* src = g.slabs + z * slab + so;
    if (svec) {
      const int4 t = *reinterpret_cast<const int4*>(src);
      a4[0] += t.x; a4[1] += t.y; a4[2] += t.z; a4[3] += t.w;
    } else {
      for (int e = 0; e < nv; ++e) a4[e] += src[e];
    }
  }
  const int64_t o = bz * g.stride_c + mm * g.ldc + n4;
  if (g.acc_out != nullptr)
    for (int e = 0; e < nv; ++e) reinterpret_cast<int32_t*>(g.acc_out)[o + e] = a4[e];
  if constexpr (EPI == 3) {
    for (int e = 0; e < nv; ++e) reinterpret_cast<int32_t*>(g.c)[o + e] = a4[e];
  } else {
    const float s_row = g.row_scale ? g.row_scale[bz * g.stride_rs + mm] : 1.0f;
    const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
    float f[4];
#pragma unroll
    for (int e = 0; e < 4; ++e)
      f[e] = dequant_value<EPI, COL_FIRST>(a4[e], s_row, (cs != nullptr && e < nv) ? cs[n4 + e] : 1.0f);
    const bool cvec = nv == 4 && (g.ldc % 4) == 0 && (g.stride_c % 4) == 0;
    if constexpr (kOutBf16) {
      uint16_t* c = reinterpret_cast<uint16_t*>(g.c) + o;
      if (cvec && ((uintptr_t)g.c % 8) == 0) {
        uint2 w;
        w.x = (uint32_t)bf16_bits(f[0]) | ((uint32_t)bf16_bits(f[1]) << 16);
        w.y = (uint32_t)bf16_bits(f[2]) | ((uint32_t)bf16_bits(f[3]) << 16);
        *reinterpret_cast<uint2*>(c) = w;
      } else {
        for (int e = 0; e < nv; ++e) c[e] = bf16_bits(f[e]);
      }
    } else {
      float* c = reinterpret_cast<float*>(g.c) + o;
      if (cvec && ((uintptr_t)g.c % 16) == 0) *reinterpret_cast<float4*>(c) = make_float4(f[0], f[1], f[2], f[3]);
      else for (int e = 0; e < nv; ++e) c[e] = f[e];
    }
  }
}

// Reference-shaped fallback for operands the MFMA kernel cannot load with 16-byte
// vectors (contraction length or leading dimension not a multiple of 16, unaligned
// base).  One thread per output element; correct for any shape.  DEC_A/DEC_B decode one
// operand byte to a float (exact for int8 and fp8).
template <class DecA, class DecB, bool INT_ACC>
__global__ void gemm_simple_kernel(const GemmArgs g) {
  const int64_t nn = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t mm = blockIdx.y;
  const int64_t bz = blockIdx.z;
  if (nn >= g.n) return;
  const uint8_t* A = g.a + bz * g.stride_a + mm * g.lda;
  const uint8_t* B = g.b + bz * g.stride_b + nn * g.ldb;
  const int64_t o = bz * g.stride_c + mm * g.ldc + nn;
  float facc;
  if constexpr (INT_ACC) {
    int acc = 0;
    for (int64_t kk = 0; kk < g.k; ++kk) acc += (int)(int8_t)A[kk] * (int)(int8_t)B[kk];
    if (g.acc_out) reinterpret_cast<int32_t*>(g.acc_out)[o] = acc;
    if (g.out_dtype == AQTX_I32) {
      reinterpret_cast<int32_t*>(g.c)[o] = acc;
      return;
    }
    facc = (float)acc;
  } else {
    facc = 0.0f;
    for (int64_t kk = 0; kk < g.k; ++kk) facc = fmaf(DecA::decode(A[kk]), DecB::decode(B[kk]), facc);
    if (g.acc_out) reinterpret_cast<float*>(g.acc_out)[o] = facc;
  }
  float f = rnd(facc, g.dq_bf16);
  const float* rs = g.row_scale ? g.row_scale + bz * g.stride_rs : nullptr;
  const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
  if (g.col_first) {
    if (cs) f = rnd(f * cs[nn], g.p1_bf16);
    if (rs) f = rnd(f * rs[mm], g.p2_bf16);
  } else {
    if (rs) f = rnd(f * rs[mm], g.p1_bf16);
    if (cs) f = rnd(f * cs[nn], g.p2_bf16);
  }
  f = rnd(f, g.dq_bf16);
  if (g.out_dtype == AQTX_BF16) reinterpret_cast<uint16_t*>(g.c)[o] = bf16_bits(f);
  else reinterpret_cast<float*>(g.c)[o] = f;
}

struct DecI8 {
  static __device__ __forceinline__ float decode(uint8_t v) { return (float)(int8_t)v; }
};
struct DecE4M3 {  // e4m3fn: bias 7, no infinities
  static __device__ __forceinline__ float decode(uint8_t v) {
    const int e = (v >> 3) & 15, m = v & 7;
    float f = e == 0 ? ldexpf((float)m, -9) : ldexpf((float)(8 + m), e - 10);
    if (e == 15 && m == 7) f = __builtin_nanf("");
    return (v & 0x80) ? -f : f;
  }
};
struct DecE5M2 {  // e5m2: bias 15, IEEE-like
  static __device__ __forceinline__ float decode(uint8_t v) {
    const int e = (v >> 2) & 31, m = v & 3;
    float f = e == 0 ? ldexpf((float)m, -16) : ldexpf((float)(4 + m), e - 17);
    if (e == 31) f = m ? __builtin_nanf("") : __builtin_inff();
    return (v & 0x80) ? -f : f;
  }
};

// Fills GemmArgs from a validated plan.
inline GemmArgs make_gemm_args(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                               const float* col_scale, void* c, void* acc_out) {
  GemmArgs g{};
  g.a = reinterpret_cast<const uint8_t*>(a);
  g.b = reinterpret_cast<const uint8_t*>(b);
  g.row_scale = row_scale; g.col_scale = col_scale;
  g.c = c; g.acc_out = acc_out;
  g.m = p->m; g.n = p->n; g.k = p->k;
  g.lda = p->lda; g.ldb = p->ldb; g.ldc = p->ldc;
  g.stride_a = p->stride_a; g.stride_b = p->stride_b; g.stride_c = p->stride_c;
  g.stride_rs = p->row_scale_stride_b; g.stride_cs = p->col_scale_stride_b;
  g.out_dtype = p->out_dtype;
  g.dq_bf16 = p->dequant_dtype == AQTX_BF16;
  g.col_first = p->scale_order == AQTX_SCALE_COL_THEN_ROW;
  {
    // jnp promotion, product by product: bf16 * bf16 -> bf16, anything with f32 -> f32 for good.
    // A missing scale multiplies by 1 and changes nothing, so only its dtype's effect on the
    // promotion matters; it is taken as given.
    const bool first_bf = (g.col_first ? p->col_scale_dtype : p->row_scale_dtype) == AQTX_BF16;
    const bool second_bf = (g.col_first ? p->row_scale_dtype : p->col_scale_dtype) == AQTX_BF16;
    g.p1_bf16 = g.dq_bf16 && first_bf;
    g.p2_bf16 = g.p1_bf16 && second_bf;
  }
  g.tiles_m = (int)((p->m + BM - 1) / BM);
  g.tiles_n = (int)((p->n + BN - 1) / BN);
  g.group_offsets = p->group_offsets;
  return g;
}

inline bool gemm_vector_shape_ok(const aqtx_gemm_plan* p) {
  return (p->k % 16 == 0) && (p->lda % 16 == 0) && (p->ldb % 16 == 0) && (p->stride_a % 16 == 0) &&
         (p->stride_b % 16 == 0) && p->k > 0;
}

inline bool gemm_vector_path_ok(const aqtx_gemm_plan* p, const void* a, const void* b) {
  return gemm_vector_shape_ok(p) && ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0);
}

// Epilogue id for the (out, dequant, scale) dtype triple, or -1.
inline int gemm_epilogue_id(const aqtx_gemm_plan* p) {
  if (p->out_dtype == AQTX_I32) return 3;
  const bool first_bf = (p->scale_order == AQTX_SCALE_COL_THEN_ROW ? p->col_scale_dtype : p->row_scale_dtype) == AQTX_BF16;
  const bool second_bf = (p->scale_order == AQTX_SCALE_COL_THEN_ROW ? p->row_scale_dtype : p->col_scale_dtype) == AQTX_BF16;
  if (p->out_dtype == AQTX_BF16 && p->dequant_dtype == AQTX_BF16) return first_bf ? (second_bf ? 0 : 4) : 1;
  if (p->out_dtype == AQTX_F32 && p->dequant_dtype == AQTX_F32) return 2;  // f32 * any scale stays f32
  return -1;
}

}  // namespace

int validate_gemm_plan(const aqtx_gemm_plan* p, const char* who, bool fp8);
// gemm_mid.hip: 0 = the plan stays with the 256 x 256 kernel, 1 = the 128 x 128 kernel, S > 1 = with K in S slices
int compute_units();  // CUs of the current device (0 if it cannot be asked)
int gemm_mid_k_slices(const aqtx_gemm_plan* p);
int launch_gemm_i8_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                       const float* col_scale, void* c, int32_t* acc_out, int slices, hipStream_t st);
int launch_conv_i8_mid(const aqtx_im2col_plan* w, const aqtx_gemm_plan* p, const void* x, const void* b,
                       const float* row_scale, const float* col_scale, void* c, hipStream_t st);
int launch_gemm_fp8_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                        const float* col_scale, void* c, float* acc_out, hipStream_t st);
// the same plan contracted through bf16 (plan->accumulate == AQTX_ACC_F32)
int launch_gemm_fp8_f32sum_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                               const float* col_scale, void* c, float* acc_out, hipStream_t st);
// gemm_i8_frag.hip: the 256 x 256 kernel (8 waves, row scale first) on a fragment-ordered b
int launch_gemm_i8_frag(const aqtx_gemm_plan* p, const void* a, const void* b, const float* row_scale,
                        const float* col_scale, void* c, int32_t* acc_out, hipStream_t st);
int launch_gemm_weight_only_mid(const aqtx_gemm_plan* p, const void* a, const void* b, const float* col_scale, void* c,
                                hipStream_t st);
// gemm_wo.hip: the same contraction on 256 x 256 tiles; `workgroups` > 0: that many workgroups walk the tiles
int launch_gemm_weight_only_large(const aqtx_gemm_plan* p, const void* a, const void* b, const float* col_scale, void* c,
                                  int workgroups, hipStream_t st);

}  // namespace aqtx

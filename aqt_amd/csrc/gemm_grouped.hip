// int8 x int8/int4 contraction with one scale pair per group of the contraction axis
// (subchannel / tiled quantization): for every group g of `group` consecutive k,
//   part_g[m, n] = round( round( cast(sum_{k in g} A[m,k] B[n,k]) * s_row[g][m] ) * s_col[g][n] )
//   C[m, n]      = cast( sum_g part_g[m, n] )          (float32 accumulation in group order)
// which is what tiled_dot_general does with a quantizing inner dot_general: the tile-count axis is
// a batch axis of the inner call, every tile is dequantized (rounded to the dequant dtype) on its
// own and the tiles are summed afterwards.  Here the per-group results never leave registers.
//
// The per-group rescale is 7 vector instructions per element and group (int->float, three
// roundings to bf16, two multiplications, one addition) against one MFMA per 1024 elements and
// 32 k: with groups of 128 the kernel is bound by the vector ALU, not by the matrix cores.  On
// this device a wave issues one vector instruction every ~12 cycles however independent its
// instructions are (measured: 2 waves per SIMD reach 2.7 ns per instruction and SIMD, 4 waves
// 1.5 ns for add/mul/and and 2.3 ns for the conversions and shifts), so a kernel of this kind
// wants 4 waves per SIMD, i.e. at most 128 registers per lane, more than it wants large tiles.
//
// Two tile kernels, both with 128-byte K stages double-buffered in LDS, the group scales of a stage
// next to it in LDS (and gemm_grouped_rows_kernel, further down, for at most 64 rows of A):
//   gemm_grouped128_kernel  group = 128 (one stage per group).  Workgroup = 8 waves (4 x 2) on a
//       128 x 128 tile of C, a wave 32 x 64 = two MFMA tiles (v_mfma_i32_32x32x32_i8): 32 int32
//       accumulators of the current group and 32 float32 running sums; two workgroups per CU.
//   gemm_grouped_kernel     longer groups.  Workgroup = 8 waves (2 x 4) on 128 x 256, a wave
//       64 x 64, LDS under the XOR swizzle of the dense kernel; the rescale follows the last
//       stage of a group.
//
// Packed int4 weights (two values per byte, low nibble = even k) are unpacked in registers on their
// way to LDS: a nibble is moved to the top of its byte (value * 16) and the factor 1/16 is folded,
// exactly, into the column scale.
//
// Not used, measured: accumulating the rounded group results with v_mfma_f32_32x32x16_bf16 against
// a 0/1 selection matrix (which would save the widening and the addition) is not a correctly
// rounded float32 addition on this device: 2-10 % of random sums differ in the last bit.
#include "gemm_core.h"

namespace aqtx {
namespace {

constexpr int GM = 128;  // rows of C per workgroup; a stage is BK = 128 bytes of K
constexpr int grouped_cols(bool group128) { return group128 ? 128 : 256; }

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// Rounds a float to bf16 (ties to even) and widens it again in one instruction: the packed
// conversion of (0, x) leaves bf16(x) in the upper half of the word over a zero lower half.
template <bool kBf16>
__device__ __forceinline__ float round_wide(float x) {
  if constexpr (kBf16) {
    const bf16x2 h = __builtin_convertvector(f32x2{0.0f, x}, bf16x2);
    return __builtin_bit_cast(float, h);
  } else {
    return x;
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
  int a_even_odd8;   // A's bytes of every 8 k are stored as k 0,2,4,6,1,3,5,7 (packed B only)
  int rs_by_row;     // row_scale is [m][groups] instead of [groups][m]
};

__device__ __forceinline__ int row_swz(int row) { return (row ^ (row >> 3)) & 7; }

// EPI as in the dense kernel: 0 = bf16 out, both products rounded to bf16; 4 = bf16 out, first
// product bf16, second f32; 1 = bf16 out, products in f32; 2 = f32 out.
template <int EPI>
struct Rescale {
  static constexpr bool kOutBf16 = EPI != 2;
  static constexpr bool kP1Bf16 = EPI == 0 || EPI == 4;
  static constexpr bool kP2Bf16 = EPI == 0;
  // sum[r] += dequant(acc[r]) for registers r = 4q .. 4q+3 of NT accumulator tiles that share the
  // four column scales cs (tile t has row scale rs[t]).  Every product and the sum round on their
  // own (the library is built with floating-point contraction off, so no fused multiply-add
  // appears here); the elements go through each step together, not one after the other.
  template <int NT>
  static __device__ __forceinline__ void quarter(const v16i* const (&acc)[NT], v16f* const (&sum)[NT], const int q,
                                                 const float (&rs)[NT], const float4 cs4) {
    const float cs[4] = {cs4.x, cs4.y, cs4.z, cs4.w};
    float f[4 * NT];
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] = (float)(*acc[i >> 2])[4 * q + (i & 3)];
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] = round_wide<kOutBf16>(f[i]);
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] *= rs[i >> 2];
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] = round_wide<kP1Bf16>(f[i]);
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] *= cs[i & 3];
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) f[i] = round_wide<kP2Bf16 || kOutBf16>(f[i]);  // P2 rounding, or the tile's final cast
#pragma unroll
    for (int i = 0; i < 4 * NT; ++i) (*sum[i >> 2])[4 * q + (i & 3)] += f[i];
  }
};

// Writes registers 4q..4q+3 of a running-sum tile: four consecutive n of row mm.
template <bool kOutBf16>
__device__ __forceinline__ void store_out4(const GroupedArgs& g, const v16f& sum, int q, int64_t mm, int64_t nn, bool vec) {
  constexpr int kEsz = kOutBf16 ? 2 : 4;
  if (mm >= g.m || nn >= g.n) return;
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = round_to<kOutBf16>(sum[4 * q + e]);
  uint8_t* dst = reinterpret_cast<uint8_t*>(g.c) + (mm * g.ldc + nn) * kEsz;
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

// The group scale this thread fetches for its workgroup: thread t < GM a row scale, GM <= t <
// GM + GN a column scale.  The load is unconditional from a clamped address and nothing reads its
// result before store(): a use next to the load would wait there for every load issued before it.
template <int GN, bool PACKED>
struct ScaleFetch {
  const float* ptr;
  int64_t len;  // elements from one group's scale to the next
  float reg = 1.0f;
  bool row, inside, valid = false, active;
  int groups;
  __device__ __forceinline__ ScaleFetch(const GroupedArgs& g, int tid, int64_t m0, int64_t n0) {
    row = tid < GM;
    active = tid < GM + GN;
    const int64_t idx = row ? m0 + tid : n0 + (tid - GM);
    const int64_t n_idx = row ? g.m : g.n;
    inside = active && idx < n_idx;
    const bool by_idx = row && g.rs_by_row;  // [idx][group] instead of [group][idx]
    ptr = (row ? g.row_scale : g.col_scale) + (inside ? idx : 0) * (by_idx ? g.groups : 1);
    len = by_idx ? 1 : n_idx;
    groups = g.groups;
  }
  // called for grp = 0, 1, 2, ... in order: the pointer moves on by one group per call and stops
  // at the last group
  __device__ __forceinline__ void load(int grp) {
    valid = inside && grp < groups;
    if (active) reg = *ptr;
    if (grp + 1 < groups) ptr += len;
  }
  __device__ __forceinline__ void store(int tid, float* srow, float* scol) {
    asm volatile("" : "+v"(reg));  // keeps the arithmetic on the loaded value down here
    const float v = valid ? reg * ((PACKED && !row) ? 0.0625f : 1.0f) : 1.0f;
    if (row) srow[tid] = v;
    else if (active) scol[tid - GM] = v;
  }
};

// ---- group = 128 ---------------------------------------------------------------------------------
// LDS rows are 144 bytes apart (128 of data, 16 of padding) instead of XOR-swizzled: the 16 lanes
// of a fragment read still fall into 64 distinct banks, and every address of the loop is one of a
// few loop-invariant registers plus an immediate, which this kernel needs more than it needs
// the 12 % of LDS: it has 128 registers per lane.
//
// A stage: eight MFMAs (four 32-byte k steps x two column tiles); the staging registers (stage
// s + 1, requested during stage s - 1) go to LDS, into the buffer stage s - 1 left; the rescale of
// the group just accumulated, with the global loads of stage s + 2 issued one per quarter of it
// (issued in one burst, the loads of all waves queue up in the CU's address unit and the waves
// stand still behind them); the next group's scales go to LDS; barrier.  The other three waves of
// the SIMD fill the gaps each of these leaves.
template <int EPI, bool PACKED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4)))
void gemm_grouped128_kernel(const GroupedArgs g) {
  using R = Rescale<EPI>;
  constexpr int GN = grouped_cols(true);
  constexpr int kRow = BK + 16;
  constexpr int kATile = GM * kRow, kBTile = GN * kRow, kStage = kATile + kBTile;  // 36 KiB
  __shared__ __attribute__((aligned(1024))) uint8_t stage_mem[2 * kStage];
  __shared__ __attribute__((aligned(16))) float srow[2][GM];
  __shared__ __attribute__((aligned(16))) float scol[2][GN];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;  // 32 rows, 64 columns
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
  // The second load of an operand (rows 8 further down) has a descriptor of its own, 8 rows in: only the
  // vector offset of a buffer load is range checked, so those 8 rows cannot travel in the scalar offset
  // (rows past the operand would really be fetched), and a second vector offset would cost a register.
  const __amdgpu_buffer_rsrc_t rsrc_a8 = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(g.a + (m0 + 8) * g.lda), 0, rows_a > 8 ? (int)((rows_a - 9) * g.lda + g.k) : 0, kBufferRsrcWord3);
  const __amdgpu_buffer_rsrc_t rsrc_b8 = __builtin_amdgcn_make_buffer_rsrc(
      (void*)(g.b + (n0 + 8) * g.ldb), 0, rows_b > 8 ? (int)((rows_b - 9) * g.ldb + kb_bytes) : 0, kBufferRsrcWord3);
  // group scales: waves 0, 1 fetch the 128 row scales, waves 2, 3 the 128 column scales of the next
  // group, one per lane, through a buffer whose scalar offset selects the group.  Nothing reads the
  // result before it goes to LDS at the end of the stage: a use next to the load would wait there
  // for every load issued before it.
  const bool sc_row = wave < 2, sc_active = wave < 4;
  const int sc_idx = (tid & 127);
  const int64_t sc_len = sc_row ? g.m : g.n, sc_first = sc_row ? m0 : n0;
  const bool sc_inside = sc_active && sc_first + sc_idx < sc_len;
  const bool sc_by_idx = sc_row && g.rs_by_row;  // [row][group] instead of [group][row]
  const int64_t sc_skip = sc_first * (sc_by_idx ? g.groups : 1);
  const __amdgpu_buffer_rsrc_t rsrc_s = __builtin_amdgcn_make_buffer_rsrc(
      (void*)((sc_row ? g.row_scale : g.col_scale) + sc_skip), 0, (int)(((int64_t)g.groups * sc_len - sc_skip) * 4),
      kBufferRsrcWord3);
  const int sc_step = sc_by_idx ? 4 : (int)sc_len * 4;  // bytes from one group's scale to the next
  // lanes past the operand fetch its last scale (store_scales masks them): no address past the array
  const int sc_idx_in = sc_first + sc_idx < sc_len ? sc_idx : (int)(sc_len - 1 - sc_first);
  const int sc_voff = sc_idx_in * (sc_by_idx ? g.groups * 4 : 4);
  float sc_reg = 1.0f;
  auto load_scales = [&](int grp) {
    const int grp_c = grp < g.groups ? grp : g.groups - 1;
    if (sc_active) sc_reg = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_s, sc_voff, grp_c * sc_step, 0));
  };
  auto store_scales = [&](int grp, int buf) {
    asm volatile("" : "+v"(sc_reg));  // keeps the arithmetic on the loaded value down here
    const float v = (sc_inside && grp < g.groups) ? sc_reg * ((PACKED && !sc_row) ? 0.0625f : 1.0f) : 1.0f;
    if (sc_row) srow[buf][sc_idx] = v;
    else if (sc_active) scol[buf][sc_idx] = v;
  };

  // ---- global -> registers -> LDS (rows past the operand read as zero) ----------------------
  // A: 16 blocks of 8 rows x 128 B, two per wave.  B unpacked: 16 such blocks, two per wave.
  // B packed: a wave load covers 16 rows x 64 B, one per wave; a lane's 16 bytes become the 32
  // bytes at 32 * (lane & 3) of its row.  The two loads of an operand differ by their descriptor.
  constexpr int NLA = 2, NLB = PACKED ? 1 : 2, NL = NLA + NLB;
  v4i stg[NL];
  const int ld_a = (wave * 16 + (lane >> 3)) * (int)g.lda + (lane & 7) * 16;
  const int ld_b = PACKED ? (wave * 16 + (lane >> 2)) * (int)g.ldb + (lane & 3) * 16
                          : (wave * 16 + (lane >> 3)) * (int)g.ldb + (lane & 7) * 16;
  const int st_a = (wave * 16 + (lane >> 3)) * kRow + (lane & 7) * 16;
  const int st_b = kATile + (PACKED ? (wave * 16 + (lane >> 2)) * kRow + (lane & 3) * 32
                                    : (wave * 16 + (lane >> 3)) * kRow + (lane & 7) * 16);
  auto load_one = [&](const int j, int k0) {
    if (j < NLA) stg[j] = __builtin_amdgcn_raw_buffer_load_b128(j == 0 ? rsrc_a : rsrc_a8, ld_a, k0, 0);
    else if constexpr (PACKED) stg[j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, ld_b, k0 / 2, 0);
    else stg[j] = __builtin_amdgcn_raw_buffer_load_b128(j == NLA ? rsrc_b : rsrc_b8, ld_b, k0, 0);
  };
  auto store_stage = [&](const int stage_base) {
    uint8_t* st = stage_mem + stage_base;
#pragma unroll
    for (int j = 0; j < NLA; ++j) *reinterpret_cast<v4i*>(st + st_a + j * 8 * kRow) = stg[j];
    if constexpr (PACKED) {
      v4i lo, hi;
      unpack_i4x32(stg[NLA], lo, hi, g.a_even_odd8);
      *reinterpret_cast<v4i*>(st + st_b) = lo;
      *reinterpret_cast<v4i*>(st + st_b + 16) = hi;
    } else {
#pragma unroll
      for (int j = 0; j < NLB; ++j) *reinterpret_cast<v4i*>(st + st_b + j * 8 * kRow) = stg[NLA + j];
    }
  };

  // fragment of k step ks: 16 bytes at 32 ks + 16 lh of row lr of the 32-row block
  const int a_off = (wm * 32 + lr) * kRow + lh * 16;
  const int b_off = kATile + (wn * 64 + lr) * kRow + lh * 16;
  const int rs_off = wm * 32 + lr, cs_off = wn * 64 + 4 * lh;

  v16i acc[2];
  v16f sum[2];
#pragma unroll
  for (int r = 0; r < 16; ++r) { acc[0][r] = 0; acc[1][r] = 0; sum[0][r] = 0.0f; sum[1][r] = 0.0f; }
  const v16i kZero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  const int nstages = g.groups;
  for (int j = 0; j < NL; ++j) load_one(j, 0);
  load_scales(0);
  store_stage(0);
  store_scales(0, 0);
  for (int j = 0; j < NL; ++j) load_one(j, nstages > 1 ? BK : 0);
  __syncthreads();

  // BUF (compile time) is the LDS buffer of stage s, so that every LDS address is a register plus an immediate
  auto stage = [&](const int s, auto buf_c) {
    constexpr int BUF = decltype(buf_c)::value;
    const uint8_t* st = stage_mem + BUF * kStage;
    load_scales(s + 1);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const v4i fa = *reinterpret_cast<const v4i*>(st + a_off + ks * 32);
      const v4i fb0 = *reinterpret_cast<const v4i*>(st + b_off + ks * 32);
      const v4i fb1 = *reinterpret_cast<const v4i*>(st + b_off + 32 * kRow + ks * 32);
      // the first MFMA of a group starts from a zero accumulator operand instead of zeroed registers
      acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb0, fa, ks == 0 ? kZero : acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb1, fa, ks == 0 ? kZero : acc[1], 0, 0, 0);
    }
    // Past the last stage the store and the loads are repeated harmlessly (a buffer nobody reads,
    // k offset 0) rather than branched around.
    store_stage((1 - BUF) * kStage);
    const int k_next = s + 2 < nstages ? (s + 2) * BK : 0;
    // lane holds C[m = wm*32 + lr][n = wn*64 + ni*32 + 8q + 4lh + e], register 4q + e of tile ni
    const float rs[1] = {srow[BUF][rs_off]};
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        if (ni * 4 + q < NL) load_one(ni * 4 + q, k_next);
        const v16i* const a1[1] = {&acc[ni]};
        v16f* const s1[1] = {&sum[ni]};
        R::template quarter<1>(a1, s1, q, rs, *reinterpret_cast<const float4*>(&scol[BUF][cs_off + ni * 32 + 8 * q]));
      }
    store_scales(s + 1, 1 - BUF);
    // a bare s_barrier: a __syncthreads() would also wait for the global loads just issued
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  for (int s = 0; s < nstages; s += 2) {
    stage(s, std::integral_constant<int, 0>{});
    if (s + 1 < nstages) stage(s + 1, std::integral_constant<int, 1>{});
  }

  const bool vec = (g.ldc % 4) == 0 && ((uintptr_t)g.c % 16) == 0;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      store_out4<R::kOutBf16>(g, sum[ni], q, m0 + wm * 32 + lr, n0 + wn * 64 + ni * 32 + 8 * q + 4 * lh, vec);
}

// ---- groups of 256 and more ------------------------------------------------------------------------
template <int EPI, bool PACKED>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void gemm_grouped_kernel(const GroupedArgs g) {
  using R = Rescale<EPI>;
  constexpr int GN = grouped_cols(false);
  constexpr int kATile = GM * BK, kBTile = GN * BK, kStage = kATile + kBTile;  // 48 KiB
  __shared__ __attribute__((aligned(1024))) uint8_t stage_mem[2][kStage];
  __shared__ __attribute__((aligned(16))) float srow[2][GM];
  __shared__ __attribute__((aligned(16))) float scol[2][GN];

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 2, wn = wave & 3;  // 64 rows, 64 columns
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
  // B packed: a wave load covers 16 rows x 64 B; two per wave.
  constexpr int NLA = 2, NLB = PACKED ? 2 : 4;
  // two sets of staging registers: a stage without a rescale is short, so the loads of a stage
  // are issued two stages ahead of its use and written to LDS one stage ahead
  v4i sta[2][NLA], stb[2][NLB];
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
        const int row = (wave * NLB + i) * 16 + (lane >> 2), p = lane & 3;
        v4i lo, hi;
        unpack_i4x32(stb[set][i], lo, hi, g.a_even_odd8);
        uint8_t* rowp = st + kATile + row * BK;
        *reinterpret_cast<v4i*>(rowp + (((2 * p) ^ row_swz(row)) * 16)) = lo;
        *reinterpret_cast<v4i*>(rowp + (((2 * p + 1) ^ row_swz(row)) * 16)) = hi;
      } else {
        *reinterpret_cast<v4i*>(st + kATile + (wave * NLB + i) * 1024 + lane * 16) = stb[set][i];
      }
    }
  };
  ScaleFetch<GN, PACKED> sc(g, tid, m0, n0);

  const int frag_off0 = lr * BK + ((lh ^ ((lr ^ (lr >> 3)) & 7)) * 16);
  auto frag_off = [&](int c) { return frag_off0 ^ (c * 16); };
  const int a_base = wm * 64 * BK, b_base = kATile + wn * 64 * BK;

  v16i acc[2][2];
  v16f sum[2][2];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int r = 0; r < 16; ++r) { acc[mi][ni][r] = 0; sum[mi][ni][r] = 0.0f; }
  const v16i kZero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};

  const int nstages = g.groups * g.stages_per_group;
  load_stage(0, 0);
  sc.load(0);
  store_stage(0, stage_mem[0]);
  sc.store(tid, srow[0], scol[0]);
  if (nstages > 1) load_stage(1, BK);  // set 1 holds stage 1, set 0 will take stage 2, ...
  __syncthreads();
  // one stage; `set` holds the registers of stage s + 1, the other set takes the loads of s + 2
  auto stage = [&](const int s, const int set) {
    const int grp = s / g.stages_per_group, pos = s % g.stages_per_group;
    const bool last_of_group = pos + 1 == g.stages_per_group;
    const uint8_t* st = stage_mem[s & 1];
    if (s + 2 < nstages) load_stage(set ^ 1, (s + 2) * BK);
    if (last_of_group) sc.load(grp + 1);
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      v4i fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int c = (2 * ks) ^ (4 * (i & 1));
        fa[i] = *reinterpret_cast<const v4i*>(st + a_base + i * 32 * BK + frag_off(c));
        fb[i] = *reinterpret_cast<const v4i*>(st + b_base + i * 32 * BK + frag_off(c));
      }
      // the first MFMA of a group starts from a zero accumulator operand instead of zeroed registers
      const bool fresh = ks == 0 && pos == 0;
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int ni = 0; ni < 2; ++ni) {
          if (fresh) acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], kZero, 0, 0, 0);
          else acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
        }
    }
    if (last_of_group) {
      // lane holds C[m = wm*64 + mi*32 + lr][n = wn*64 + ni*32 + 8q + 4lh + e], register 4q + e
      const int buf = grp & 1;
      const float rs[2] = {srow[buf][wm * 64 + lr], srow[buf][wm * 64 + 32 + lr]};
#pragma unroll
      for (int ni = 0; ni < 2; ++ni)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const v16i* const a2[2] = {&acc[0][ni], &acc[1][ni]};
          v16f* const s2[2] = {&sum[0][ni], &sum[1][ni]};
          R::template quarter<2>(a2, s2, q, rs, *reinterpret_cast<const float4*>(&scol[buf][wn * 64 + ni * 32 + 8 * q + 4 * lh]));
        }
    }
    // the registers of stage s + 1 (requested a whole stage ago) go to the buffer stage s - 1 left;
    // the barrier is a bare s_barrier: a __syncthreads() would also wait for the loads of s + 2
    if (s + 1 < nstages) store_stage(set, stage_mem[(s + 1) & 1]);
    if (last_of_group) sc.store(tid, srow[(grp + 1) & 1], scol[(grp + 1) & 1]);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  };
  for (int s = 0; s < nstages; s += 2) {
    stage(s, 1);
    if (s + 1 < nstages) stage(s + 1, 0);
  }

  const bool vec = (g.ldc % 4) == 0 && ((uintptr_t)g.c % 16) == 0;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int ni = 0; ni < 2; ++ni)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        store_out4<R::kOutBf16>(g, sum[mi][ni], q, m0 + wm * 64 + mi * 32 + lr, n0 + wn * 64 + ni * 32 + 8 * q + 4 * lh, vec);
}

// [n][k] int4 values in int8 bytes -> [n][k/2] packed, low nibble = even k.
__global__ void pack_i4_kernel(const int8_t* src, uint8_t* dst, int64_t count2) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= count2) return;
  const uint32_t lo = (uint32_t)src[2 * i] & 0xFu, hi = (uint32_t)src[2 * i + 1] & 0xFu;
  dst[i] = (uint8_t)(lo | (hi << 4));
}

// ---- at most 64 rows of A (serving with a frozen subchannel weight) ----------------------------------
// The tile kernels above rescale a 128-row tile of C per group whatever m is: with a handful of tokens
// almost all of that vector work is spent on rows that do not exist (measured: 100 us for 1..64 tokens
// against 2048 x 8192 x 28672's packed weight, 15 % of what the weight stream alone would take).  Here a
// wave owns 16 rows of B and all tokens (MB blocks of 16) for all of K, in group order, so the running sums
// add up in the order of the tile kernels: v_mfma_i32_16x16x64_i8 with the activations as the first
// operand leaves a lane with tokens 4c .. 4c + 3 (c = lane / 16) of column lane % 16, i.e. four row scales
// and one column scale per lane and group.  A group of 128 k is one 16-byte load per lane of a packed
// weight row (two of an int8 one), requested eight groups ahead, straight from global memory into the MFMA
// operand.  The activations are shared by the NW waves of a workgroup: chunks of four groups go through
// LDS, double buffered (two with 64 tokens; every wave reading all of them from L2 instead cost as much again as the weight
// stream at 8 tokens and eight times that at 64); rows are 528 bytes apart, so that the 16 lanes of one
// operand read hit distinct banks; the chunk's row scales travel with it, as [group][token].
constexpr int rows_chunk_groups(int mb) { return mb == 4 ? 2 : 4; }  // 64 tokens: half the chunk, the same LDS

// MB: token blocks of a wave; TS: waves that share 16 rows of B, each with MB token blocks of its own (more
// waves per SIMD for the vector work of many tokens, at the price of TS requests per weight fragment).
template <int EPI, bool PACKED, int MB, int TS, int NW>
__global__ __launch_bounds__(NW * 64) void gemm_grouped_rows_kernel(const GroupedArgs g) {
  using R = Rescale<EPI>;
  constexpr int MT = 16 * MB * TS;      // tokens of the workgroup
  constexpr int CG = rows_chunk_groups(MB * TS);  // groups per activation chunk
  constexpr int kPitch = CG * 128 + 16;
  constexpr int NT = NW * 64;
  constexpr int PPC = CG * 8;           // 16-byte pieces of one token's chunk
  constexpr int XL = MT * PPC / NT;     // 16-byte activation loads per thread and chunk
  static_assert(XL >= 1 && MT * PPC % NT == 0, "chunk loads divide among the threads");
  extern __shared__ __attribute__((aligned(16))) uint8_t rows_lds[];
  uint8_t* xbuf = rows_lds;                                                  // [2][MT][kPitch]
  float* srow = reinterpret_cast<float*>(rows_lds + 2 * MT * kPitch);        // [2][CG][MT]
  static_assert(CG * MT <= NT, "one row scale per thread and chunk");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const int n0 = ((int)blockIdx.x * (NW / TS) + wave / TS) * 16;
  const int tok0 = (wave % TS) * MB * 16;  // first token of this wave
  const int kb = PACKED ? (int)(g.k / 2) : (int)g.k;
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      (void*)g.a, 0, (int)((g.m - 1) * g.lda + g.k), kBufferRsrcWord3);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      (void*)g.b, 0, (int)((g.n - 1) * g.ldb + kb), kBufferRsrcWord3);
  constexpr int kOutside = 0x7FFFFFF0;
  // lane (r, c): weight row n0 + r, bytes 16 c (packed: k 32 c .. 32 c + 31 of the group) or 32 c (int8:
  // the same k); the activations of token r, the same k: 32 bytes
  constexpr int WL = PACKED ? 1 : 2;
  const int wrow = n0 + r;
  const int woff = wrow < g.n ? wrow * (int)g.ldb + c * (PACKED ? 16 : 32) : kOutside;
  const int ncol = wrow < g.n ? wrow : (int)g.n - 1;
  const float cfold = PACKED ? 0.0625f : 1.0f;  // packed nibbles are unpacked to 16 * value
  const int nchunks = (g.groups + CG - 1) / CG;

  // activation chunk: load j of a thread is the 16-byte piece (tid + j NT) % PPC of token (tid + j NT) / PPC;
  // and, for the first CG * MT threads, the row scale of token tid % MT in group tid / MT of the chunk.
  // Chunk j waits in register set j % 2 from its request, two trips ahead of the trip that reads it (one trip is
  // shorter than a round trip to L2 under load), until the trip before that one stores it to LDS.
  v4i xs[2][XL];
  float rs_reg[2] = {1.0f, 1.0f};
  bool rs_ok[2] = {false, false};  // applied when the value goes to LDS: a use next to the load would wait for it there
  auto request_x = [&](const int set, int ch) {
    {
      const int grp = ch * CG + tid / MT, t = tid % MT;
      rs_ok[set] = tid < CG * MT && t < g.m && grp < g.groups;
      const int64_t at = g.rs_by_row ? (int64_t)t * g.groups + grp : (int64_t)grp * g.m + t;
      rs_reg[set] = g.row_scale[rs_ok[set] ? at : 0];
    }
#pragma unroll
    for (int j = 0; j < XL; ++j) {
      const int id = tid + j * NT, t = id / PPC, piece = id % PPC;
      const bool ok = t < g.m && ch * CG * 128 + piece * 16 < (int)g.k && ch < nchunks;
      xs[set][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, ok ? t * (int)g.lda + piece * 16 : kOutside,
                                                         ok ? ch * CG * 128 : 0, 0);
    }
  };
  auto store_x = [&](const int set, const int buf) {
    if (tid < CG * MT) srow[buf * CG * MT + tid] = rs_ok[set] ? rs_reg[set] : 1.0f;
#pragma unroll
    for (int j = 0; j < XL; ++j) {
      const int id = tid + j * NT, t = id / PPC, piece = id % PPC;
      *reinterpret_cast<v4i*>(xbuf + (buf * MT + t) * kPitch + piece * 16) = xs[set][j];
    }
  };
  constexpr int WD = 8;  // groups of weights (and column scales) requested ahead: about 2 us of a wave's work
  static_assert(WD % CG == 0 && (WD / CG) % 2 == 0, "a round of WD groups is an even number of chunks");
  v4i wf[WD][WL];
  float cs[WD];
  auto request_w = [&](const int u, int grp) {
    const int gc = grp < g.groups ? grp : g.groups - 1;  // past the end: the last group again, never used
#pragma unroll
    for (int j = 0; j < WL; ++j)
      wf[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, woff, gc * (PACKED ? 64 : 128) + j * 16, 0);
    cs[u] = g.col_scale[(int64_t)gc * g.n + ncol];
  };

  float sum[MB][4];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int e = 0; e < 4; ++e) sum[mb][e] = 0.0f;

  // Chunk 1 is requested ahead of the first weights on purpose: the compiler sizes the wait in front of the
  // loop's first store of a chunk for the fewest requests that can lie behind that chunk's on any path into
  // the loop, and with chunk 1 requested last here that wait also covered the weights just requested (one
  // full memory latency per round of the loop).
  request_x(0, 0);
  request_x(1, 1);
#pragma unroll
  for (int u = 0; u < WD; ++u) request_w(u, u);
  store_x(0, 0);
  request_x(0, 2);
  __syncthreads();
  const int x_off = (tok0 + r) * kPitch + c * 32;
  // a round = WD groups = WD / CG chunks (an even number: the LDS buffer of a chunk is a compile-time
  // constant); a last round that is not full runs on clamped requests and skips the sums
  for (int ch0 = 0; ch0 < nchunks; ch0 += WD / CG) {
#pragma unroll
  for (int cc = 0; cc < WD / CG; ++cc) {
    const int ch = ch0 + cc;
    const uint8_t* xb = xbuf + (cc & 1) * MT * kPitch + x_off;
#pragma unroll
    for (int uu = 0; uu < CG; ++uu) {
      const int u = cc * CG + uu;
      const int grp = ch * CG + uu;
      v4i wlo, whi;
      if constexpr (PACKED) {
        unpack_i4x32(wf[u][0], wlo, whi, g.a_even_odd8);
      } else {
        wlo = wf[u][0]; whi = wf[u][1];
      }
      const float csv = cs[u] * cfold;
      request_w(u, grp + WD);  // the registers of this group are free again
      v4i acc[MB];
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const v4i x0 = *reinterpret_cast<const v4i*>(xb + mb * 16 * kPitch + uu * 128);
        const v4i x1 = *reinterpret_cast<const v4i*>(xb + mb * 16 * kPitch + uu * 128 + 16);
        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x0, wlo, v4i{0, 0, 0, 0}, 0, 0, 0);
        acc[mb] = __builtin_amdgcn_mfma_i32_16x16x64_i8(x1, whi, acc[mb], 0, 0, 0);
      }
      if (grp < g.groups) {
        // every product and the sum round on their own, as in Rescale<EPI>::quarter
        float f[MB][4];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const float4 rs4 = *reinterpret_cast<const float4*>(&srow[((cc & 1) * CG + uu) * MT + tok0 + mb * 16 + 4 * c]);
          const float rs[4] = {rs4.x, rs4.y, rs4.z, rs4.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) f[mb][e] = round_wide<R::kOutBf16>((float)acc[mb][e]);
#pragma unroll
          for (int e = 0; e < 4; ++e) f[mb][e] = round_wide<R::kP1Bf16>(f[mb][e] * rs[e]);
#pragma unroll
          for (int e = 0; e < 4; ++e) f[mb][e] = round_wide<R::kP2Bf16 || R::kOutBf16>(f[mb][e] * csv);
#pragma unroll
          for (int e = 0; e < 4; ++e) sum[mb][e] += f[mb][e];
        }
      }
    }
    // chunk ch + 1 (in registers since the trip before last) goes to the other buffer, which every wave left
    // before the barrier that ended chunk ch - 1; chunk ch + 3 is requested into the registers it leaves
    store_x((cc + 1) & 1, (cc + 1) & 1);
    request_x((cc + 1) & 1, ch + 3);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
  }
  }
  if (wrow >= g.n) return;
#pragma unroll
  for (int mb = 0; mb < MB; ++mb)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int t = tok0 + mb * 16 + 4 * c + e;
      if (t < g.m) {
        const float o = round_to<R::kOutBf16>(sum[mb][e]);
        if constexpr (R::kOutBf16) reinterpret_cast<uint16_t*>(g.c)[(int64_t)t * g.ldc + wrow] = bf16_bits(o);
        else reinterpret_cast<float*>(g.c)[(int64_t)t * g.ldc + wrow] = o;
      }
    }
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
  const bool group128 = p->group == 128;
  const int GN = grouped_cols(group128);
  AQTX_REQUIRE(!group128 || (p->k / 128) * (p->m > p->n ? p->m : p->n) * 4 < (1ll << 31),
               "aqtx_gemm_i8_grouped: a scale array of more than 2 GiB");
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
  AQTX_REQUIRE(p->a_k_order == AQTX_K_NATURAL || (p->a_k_order == AQTX_K_EVEN_ODD8 && packed),
               "aqtx_gemm_i8_grouped: a_k_order must be AQTX_K_NATURAL, or AQTX_K_EVEN_ODD8 with a packed int4 b");
  g.a_even_odd8 = p->a_k_order == AQTX_K_EVEN_ODD8;
  g.rs_by_row = p->row_scale_by_row != 0;
  int epi;
  if (p->out_dtype == AQTX_F32) epi = 2;
  else if (p->row_scale_dtype != AQTX_BF16) epi = 1;
  else epi = p->col_scale_dtype == AQTX_BF16 ? 0 : 4;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  // a handful of rows: one wave per 16 rows of b, no tile of C padded to 128 rows
  const int mb = (int)((p->m + 15) / 16), mbt = mb == 3 ? 4 : mb;  // token blocks: 1, 2 or 4
  const size_t rows_lds = (size_t)2 * 16 * mbt * (rows_chunk_groups(mbt) * 128 + 16) +
                          (size_t)2 * rows_chunk_groups(mbt) * 16 * mbt * sizeof(float);
  if (group128 && p->m <= 64 && p->m * p->lda < (1ll << 31) && p->n * p->ldb < (1ll << 31) && p->tuning != 128) {
    // 8 waves per workgroup where that still gives every CU one, else 4; from 17 tokens on two waves share
    // their 16 rows of b and take half of the token blocks each
    const int ts = mbt >= 2 ? 2 : 1;
    const int nw = (p->n * ts + 127) / 128 >= 200 ? 8 : 4;
    const int rows_per_wg = 16 * nw / ts;
    const dim3 rgrid((unsigned)((p->n + rows_per_wg - 1) / rows_per_wg));
#define AQTX_ROWS_MB(E, P, W)                                                                        \
  do {                                                                                              \
    if (mbt == 1) gemm_grouped_rows_kernel<E, P, 1, 1, W><<<rgrid, W * 64, rows_lds, st>>>(g);      \
    else if (mbt == 2) gemm_grouped_rows_kernel<E, P, 1, 2, W><<<rgrid, W * 64, rows_lds, st>>>(g); \
    else gemm_grouped_rows_kernel<E, P, 2, 2, W><<<rgrid, W * 64, rows_lds, st>>>(g);               \
  } while (0)
#define AQTX_ROWS(E)                                                                            \
  do {                                                                                          \
    if (packed) { if (nw == 8) AQTX_ROWS_MB(E, true, 8); else AQTX_ROWS_MB(E, true, 4); }        \
    else { if (nw == 8) AQTX_ROWS_MB(E, false, 8); else AQTX_ROWS_MB(E, false, 4); }             \
  } while (0)
    switch (epi) {
      case 0: AQTX_ROWS(0); break;
      case 1: AQTX_ROWS(1); break;
      case 2: AQTX_ROWS(2); break;
      default: AQTX_ROWS(4); break;
    }
#undef AQTX_ROWS
#undef AQTX_ROWS_MB
    AQTX_HIP_CHECK_LAUNCH("gemm_grouped_rows_kernel");
    return 0;
  }
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n));
#define AQTX_LAUNCH(E)                                                                      \
  do {                                                                                     \
    if (packed && group128) gemm_grouped128_kernel<E, true><<<grid, 512, 0, st>>>(g);       \
    else if (group128) gemm_grouped128_kernel<E, false><<<grid, 512, 0, st>>>(g);           \
    else if (packed) gemm_grouped_kernel<E, true><<<grid, 512, 0, st>>>(g);                 \
    else gemm_grouped_kernel<E, false><<<grid, 512, 0, st>>>(g);                            \
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

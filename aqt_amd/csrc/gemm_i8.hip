// int8 x int8 -> int32 contraction on gfx950 MFMA with the dequantisation fused
// in the epilogue.
//
// C[m, n] = dequant( sum_k A[m, k] * B[n, k] ): both operands carry the
// contraction axis contiguously (the quantize kernels write whichever layout the
// consumer needs), so every lane feeds v_mfma_i32_32x32x32_i8 with 16 contiguous
// bytes per operand.
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
#include "common.h"

namespace aqtx {
namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct GemmArgs {
  const int8_t* a;
  const int8_t* b;
  const float* row_scale;
  const float* col_scale;
  void* c;
  int32_t* acc_out;
  int64_t m, n, k;
  int64_t lda, ldb, ldc;
  int64_t stride_a, stride_b, stride_c, stride_rs, stride_cs;
  int tiles_m, tiles_n;
  int out_dtype;  // AQTX_BF16 | AQTX_F32 | AQTX_I32
  int dq_bf16;    // dequant dtype is bf16
  int sc_bf16;    // scale dtype is bf16
  int col_first;  // scale order
};

constexpr int BM = 256, BN = 256, BK = 128;
constexpr int kStageBytes = (BM + BN) * BK;       // 65536
constexpr int kEpiRowBytes = 256 + 8;             // padded row of one wave's 128-row region
constexpr int kEpiWaveBytes = 128 * kEpiRowBytes; // 33792
constexpr int kLdsBytes = 4 * kEpiWaveBytes > 2 * kStageBytes ? 4 * kEpiWaveBytes : 2 * kStageBytes;

__device__ __forceinline__ float rnd(float x, int bf) { return bf ? round_bf16(x) : x; }

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

__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1)))
void gemm_i8_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(16))) uint8_t lds[kLdsBytes];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 31, lh = lane >> 5;

  int tm, tn;
  tile_of_block(blockIdx.x, g.tiles_m, g.tiles_n, tm, tn);
  const int64_t bz = blockIdx.y;
  const int64_t m0 = (int64_t)tm * BM, n0 = (int64_t)tn * BN;
  const int8_t* A = g.a + bz * g.stride_a;
  const int8_t* B = g.b + bz * g.stride_b;

  // ---- global -> register staging: thread owns chunk (tid&7) of rows (tid>>3)+32*i
  const int gc = tid & 7, gr = tid >> 3;
  const int gf0 = (gr ^ (gr >> 3)) & 7;
  uint4 stage_a[8], stage_b[8];

  auto load_global = [&](int64_t k0) {
    const int64_t kb = k0 + gc * 16;
    const bool kok = kb < g.k;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t ra = m0 + gr + 32 * i, rb = n0 + gr + 32 * i;
      stage_a[i] = (kok && ra < g.m) ? *reinterpret_cast<const uint4*>(A + ra * g.lda + kb)
                                     : make_uint4(0, 0, 0, 0);
      stage_b[i] = (kok && rb < g.n) ? *reinterpret_cast<const uint4*>(B + rb * g.ldb + kb)
                                     : make_uint4(0, 0, 0, 0);
    }
  };
  auto store_lds = [&](int stage) {
    uint8_t* sa = lds + stage * kStageBytes;
    uint8_t* sb = sa + BM * BK;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = gr + 32 * i;
      const int sw = (gc ^ gf0 ^ (4 * (i & 1))) * 16;
      *reinterpret_cast<uint4*>(sa + row * BK + sw) = stage_a[i];
      *reinterpret_cast<uint4*>(sb + row * BK + sw) = stage_b[i];
    }
  };

  // ---- per-lane swizzled fragment offsets: chunk (2*ks + lh) ^ f(row)
  const int lf0 = (lr ^ (lr >> 3)) & 7;
  int frag_off[8];
#pragma unroll
  for (int cidx = 0; cidx < 8; ++cidx) frag_off[cidx] = lr * BK + ((lh ^ lf0 ^ cidx) * 16);
  const int a_base = wm * 128 * BK;            // rows of the A tile this wave needs
  const int b_base = BM * BK + wn * 128 * BK;  // rows of the B tile

  v16i acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;

  const int KT = (int)((g.k + BK - 1) / BK);
  load_global(0);
  store_lds(0);
  __syncthreads();

  for (int kt = 0; kt < KT; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < KT) load_global((int64_t)(kt + 1) * BK);
    const uint8_t* st = lds + cur * kStageBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      v4i fa[4], fb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int cidx = (2 * ks) ^ (4 * (i & 1));
        fa[i] = *reinterpret_cast<const v4i*>(st + a_base + i * 32 * BK + frag_off[cidx]);
        fb[i] = *reinterpret_cast<const v4i*>(st + b_base + i * 32 * BK + frag_off[cidx]);
      }
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[ni], fa[mi], acc[mi][ni], 0, 0, 0);
    }
    if (kt + 1 < KT) store_lds(cur ^ 1);
    __syncthreads();
  }

  // ---- epilogue ---------------------------------------------------------------
  // lane holds C[m = mrow0 + mi*32 + lr][n = ncol0 + ni*32 + 8*q + 4*lh + e], e = 0..3, reg = 4*q+e
  const int64_t mrow0 = m0 + wm * 128, ncol0 = n0 + wn * 128;

  if (g.acc_out != nullptr || g.out_dtype == AQTX_I32) {
    int32_t* dst = g.acc_out != nullptr ? g.acc_out : reinterpret_cast<int32_t*>(g.c);
    dst += bz * g.stride_c;
#pragma unroll
    for (int mi = 0; mi < 4; ++mi) {
      const int64_t mm = mrow0 + mi * 32 + lr;
#pragma unroll
      for (int ni = 0; ni < 4; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int64_t nn = ncol0 + ni * 32 + 8 * (r >> 2) + 4 * lh + (r & 3);
          if (mm < g.m && nn < g.n) dst[mm * g.ldc + nn] = acc[mi][ni][r];
        }
    }
    if (g.out_dtype == AQTX_I32) return;
  }

  const float* rs = g.row_scale ? g.row_scale + bz * g.stride_rs : nullptr;
  const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
  const int pbf = g.dq_bf16 & g.sc_bf16;
  float rscale[4];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const int64_t mm = mrow0 + mi * 32 + lr;
    rscale[mi] = (rs && mm < g.m) ? rs[mm] : 1.0f;
  }
  auto dequant = [&](int accv, float s_row, float s_col) {
    float f = rnd((float)accv, g.dq_bf16);
    if (g.col_first) {
      if (cs) f = rnd(f * s_col, pbf);
      if (rs) f = rnd(f * s_row, pbf);
    } else {
      if (rs) f = rnd(f * s_row, pbf);
      if (cs) f = rnd(f * s_col, pbf);
    }
    return rnd(f, g.dq_bf16);
  };

  uint8_t* region = lds + wave * kEpiWaveBytes;
  const bool out_bf16 = g.out_dtype == AQTX_BF16;
  // bf16: one pass over the 4 n-tiles (128 cols x 2 B = 256 B rows);
  // f32 : two passes of 2 n-tiles (64 cols x 4 B = 256 B rows).
  const int npass = out_bf16 ? 1 : 2;
  const int ni_per_pass = out_bf16 ? 4 : 2;
  for (int pass = 0; pass < npass; ++pass) {
#pragma unroll
    for (int nj = 0; nj < 4; ++nj) {
      if (nj >= ni_per_pass) continue;
      // static register indexing: select the tile with a compile-time switch
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int ncol_local = nj * 32 + 8 * q + 4 * lh;  // within the pass
        float csv[4] = {1.0f, 1.0f, 1.0f, 1.0f};
        {
          const int64_t nn = ncol0 + (pass * ni_per_pass) * 32 + ncol_local;
          if (cs) {
#pragma unroll
            for (int e = 0; e < 4; ++e) csv[e] = (nn + e < g.n) ? cs[nn + e] : 1.0f;
          }
        }
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
          float o[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int av = (pass == 0) ? acc[mi][nj][4 * q + e]
                                       : acc[mi][(nj + 2) & 3][4 * q + e];
            o[e] = dequant(av, rscale[mi], csv[e]);
          }
          uint8_t* p = region + (mi * 32 + lr) * kEpiRowBytes;
          if (out_bf16) {
            uint2 w;
            w.x = (uint32_t)bf16_bits(o[0]) | ((uint32_t)bf16_bits(o[1]) << 16);
            w.y = (uint32_t)bf16_bits(o[2]) | ((uint32_t)bf16_bits(o[3]) << 16);
            *reinterpret_cast<uint2*>(p + ncol_local * 2) = w;
          } else {
            *reinterpret_cast<float2*>(p + ncol_local * 4) = make_float2(o[0], o[1]);
            *reinterpret_cast<float2*>(p + ncol_local * 4 + 8) = make_float2(o[2], o[3]);
          }
        }
      }
    }
    __syncthreads();
    // read back: lane -> 16-byte chunk (lane&15) of row (lane>>4) + 4*it
    const int esz = out_bf16 ? 2 : 4;
    const int cols_per_chunk = 16 / esz;
    const int64_t ncol_pass0 = ncol0 + (int64_t)pass * ni_per_pass * 32;
    uint8_t* cbase = reinterpret_cast<uint8_t*>(g.c) + bz * g.stride_c * esz;
    for (int it = 0; it < 32; ++it) {
      const int row = (lane >> 4) + 4 * it;
      const int chunk = lane & 15;
      const int64_t mm = mrow0 + row;
      const int64_t nn = ncol_pass0 + chunk * cols_per_chunk;
      const uint2 lo = *reinterpret_cast<const uint2*>(region + row * kEpiRowBytes + chunk * 16);
      const uint2 hi = *reinterpret_cast<const uint2*>(region + row * kEpiRowBytes + chunk * 16 + 8);
      if (mm < g.m && nn < g.n) {
        uint8_t* dst = cbase + (mm * g.ldc + nn) * esz;
        if (nn + cols_per_chunk <= g.n && ((g.ldc * esz) % 16) == 0) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(lo.x, lo.y, hi.x, hi.y);
        } else {
          const uint32_t w[4] = {lo.x, lo.y, hi.x, hi.y};
          const int nv = (int)(g.n - nn) < cols_per_chunk ? (int)(g.n - nn) : cols_per_chunk;
          for (int e = 0; e < nv; ++e) {
            if (out_bf16)
              reinterpret_cast<uint16_t*>(dst)[e] = (uint16_t)(w[e >> 1] >> (16 * (e & 1)));
            else
              reinterpret_cast<uint32_t*>(dst)[e] = w[e];
          }
        }
      }
    }
    __syncthreads();
  }
}

// Reference-shaped fallback for operands the MFMA kernel cannot load with 16-byte
// vectors (contraction length or leading dimension not a multiple of 16, unaligned
// base).  One thread per output element; correct for any shape.
__global__ void gemm_i8_simple_kernel(const GemmArgs g) {
  const int64_t nn = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t mm = blockIdx.y;
  const int64_t bz = blockIdx.z;
  if (nn >= g.n) return;
  const int8_t* A = g.a + bz * g.stride_a + mm * g.lda;
  const int8_t* B = g.b + bz * g.stride_b + nn * g.ldb;
  int acc = 0;
  for (int64_t kk = 0; kk < g.k; ++kk) acc += (int)A[kk] * (int)B[kk];
  const int64_t o = bz * g.stride_c + mm * g.ldc + nn;
  if (g.acc_out) g.acc_out[o] = acc;
  if (g.out_dtype == AQTX_I32) {
    reinterpret_cast<int32_t*>(g.c)[o] = acc;
    return;
  }
  const int pbf = g.dq_bf16 & g.sc_bf16;
  float f = rnd((float)acc, g.dq_bf16);
  const float* rs = g.row_scale ? g.row_scale + bz * g.stride_rs : nullptr;
  const float* cs = g.col_scale ? g.col_scale + bz * g.stride_cs : nullptr;
  if (g.col_first) {
    if (cs) f = rnd(f * cs[nn], pbf);
    if (rs) f = rnd(f * rs[mm], pbf);
  } else {
    if (rs) f = rnd(f * rs[mm], pbf);
    if (cs) f = rnd(f * cs[nn], pbf);
  }
  f = rnd(f, g.dq_bf16);
  if (g.out_dtype == AQTX_BF16) reinterpret_cast<uint16_t*>(g.c)[o] = bf16_bits(f);
  else reinterpret_cast<float*>(g.c)[o] = f;
}

}  // namespace

int validate_gemm_plan(const aqtx_gemm_plan* p, const char* who, bool fp8) {
  AQTX_REQUIRE(p != nullptr, "%s: plan is NULL", who);
  AQTX_REQUIRE(p->batch >= 0 && p->m >= 0 && p->n >= 0 && p->k >= 0, "%s: negative shape", who);
  if (fp8) {
    AQTX_REQUIRE((p->a_dtype == AQTX_E4M3 || p->a_dtype == AQTX_E5M2) &&
                     (p->b_dtype == AQTX_E4M3 || p->b_dtype == AQTX_E5M2),
                 "%s: operands must be e4m3/e5m2 (got %d, %d)", who, p->a_dtype, p->b_dtype);
    AQTX_REQUIRE(p->out_dtype == AQTX_BF16 || p->out_dtype == AQTX_F32,
                 "%s: out_dtype must be bf16 or f32, got %d", who, p->out_dtype);
  } else {
    AQTX_REQUIRE((p->a_dtype == AQTX_I8 || p->a_dtype == AQTX_I4) &&
                     (p->b_dtype == AQTX_I8 || p->b_dtype == AQTX_I4),
                 "%s: operands must be int8 containers (got %d, %d)", who, p->a_dtype, p->b_dtype);
    AQTX_REQUIRE(p->out_dtype == AQTX_BF16 || p->out_dtype == AQTX_F32 || p->out_dtype == AQTX_I32,
                 "%s: out_dtype must be bf16, f32 or i32, got %d", who, p->out_dtype);
  }
  AQTX_REQUIRE(is_float_dtype(p->dequant_dtype), "%s: dequant_dtype must be bf16 or f32", who);
  AQTX_REQUIRE(is_float_dtype(p->scale_dtype), "%s: scale_dtype must be bf16 or f32", who);
  AQTX_REQUIRE(p->scale_order == AQTX_SCALE_ROW_THEN_COL || p->scale_order == AQTX_SCALE_COL_THEN_ROW,
               "%s: unknown scale_order %d", who, p->scale_order);
  AQTX_REQUIRE(p->lda >= p->k && p->ldb >= p->k && p->ldc >= p->n,
               "%s: leading dimension smaller than the row length", who);
  AQTX_REQUIRE(p->batch <= 65535 && p->m <= (int64_t)65535 * 256, "%s: shape too large for one launch", who);
  return 0;
}

}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_gemm_i8(const aqtx_gemm_plan* p, const void* a, const void* b,
                            const float* row_scale, const float* col_scale, void* c,
                            int32_t* acc_out, void* stream) {
  clear_error();
  if (int rc = validate_gemm_plan(p, "aqtx_gemm_i8", false)) return rc;
  if (p->batch == 0 || p->m == 0 || p->n == 0) return 0;
  AQTX_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "aqtx_gemm_i8: NULL buffer");
  AQTX_REQUIRE(p->out_dtype != AQTX_I32 || (row_scale == nullptr && col_scale == nullptr),
               "aqtx_gemm_i8: raw int32 output takes no scales");
  const size_t esz = p->out_dtype == AQTX_BF16 ? 2 : 4;
  AQTX_REQUIRE(((uintptr_t)c % esz) == 0, "aqtx_gemm_i8: output is not element aligned");

  GemmArgs g{};
  g.a = reinterpret_cast<const int8_t*>(a);
  g.b = reinterpret_cast<const int8_t*>(b);
  g.row_scale = row_scale; g.col_scale = col_scale;
  g.c = c; g.acc_out = acc_out;
  g.m = p->m; g.n = p->n; g.k = p->k;
  g.lda = p->lda; g.ldb = p->ldb; g.ldc = p->ldc;
  g.stride_a = p->stride_a; g.stride_b = p->stride_b; g.stride_c = p->stride_c;
  g.stride_rs = p->row_scale_stride_b; g.stride_cs = p->col_scale_stride_b;
  g.out_dtype = p->out_dtype;
  g.dq_bf16 = p->dequant_dtype == AQTX_BF16;
  g.sc_bf16 = p->scale_dtype == AQTX_BF16;
  g.col_first = p->scale_order == AQTX_SCALE_COL_THEN_ROW;
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);

  const bool vec_ok = (p->k % 16 == 0) && (p->lda % 16 == 0) && (p->ldb % 16 == 0) &&
                      ((uintptr_t)a % 16 == 0) && ((uintptr_t)b % 16 == 0) &&
                      (p->stride_a % 16 == 0) && (p->stride_b % 16 == 0) && p->k > 0;
  if (!vec_ok) {
    dim3 grid((unsigned)((p->n + 255) / 256), (unsigned)p->m, (unsigned)p->batch);
    AQTX_REQUIRE(p->m <= 65535, "aqtx_gemm_i8: m too large for the unaligned path");
    gemm_i8_simple_kernel<<<grid, 256, 0, st>>>(g);
    AQTX_HIP_CHECK_LAUNCH("gemm_i8_simple_kernel");
    return 0;
  }
  g.tiles_m = (int)((p->m + BM - 1) / BM);
  g.tiles_n = (int)((p->n + BN - 1) / BN);
  dim3 grid((unsigned)(g.tiles_m * g.tiles_n), (unsigned)p->batch);
  gemm_i8_kernel<<<grid, 256, 0, st>>>(g);
  AQTX_HIP_CHECK_LAUNCH("gemm_i8_kernel");
  return 0;
}

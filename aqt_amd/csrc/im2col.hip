// Window gather of a quantized convolution input: x [n][spatial...][c] int8 ->
// out [n * positions][taps * c], row = one output position, columns = the kernel window in the
// kernel's own (row-major) tap order with the features innermost, zeros where the window hangs over
// the padding.  It turns conv_general_dilated on the quantized values
// (aqt/jax/v2/aqt_conv_general.py:95-107) into the contraction the int8 MFMA kernel runs.
// One pass: reads of 16 bytes along the features, writes of full rows; HBM-bound by the output
// (taps times the input bytes).
#include "common.h"

namespace aqtx {
namespace {

struct Im2colArgs {
  const uint8_t* x;
  uint8_t* out;
  int64_t rows;      // n * positions
  int64_t k;         // taps * c
  int32_t c;
  int32_t in[3], ker[3], str[3], dil[3], pad[3], osz[3];  // up to three spatial axes, missing ones are 1
};

template <int VEC>
__global__ __launch_bounds__(256) void im2col_kernel(const Im2colArgs a) {
  const int64_t pieces = a.k / VEC;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.rows * pieces) return;
  const int64_t row = idx / pieces;
  const int64_t kp = (idx % pieces) * VEC;
  // row -> (image, output position); kp -> (tap, feature)
  int64_t r = row;
  const int o2 = (int)(r % a.osz[2]); r /= a.osz[2];
  const int o1 = (int)(r % a.osz[1]); r /= a.osz[1];
  const int o0 = (int)(r % a.osz[0]); r /= a.osz[0];
  const int64_t img = r;
  int64_t t = kp / a.c;
  const int ch = (int)(kp % a.c);
  const int t2 = (int)(t % a.ker[2]); t /= a.ker[2];
  const int t1 = (int)(t % a.ker[1]); t /= a.ker[1];
  const int t0 = (int)t;
  const int i0 = o0 * a.str[0] + t0 * a.dil[0] - a.pad[0];
  const int i1 = o1 * a.str[1] + t1 * a.dil[1] - a.pad[1];
  const int i2 = o2 * a.str[2] + t2 * a.dil[2] - a.pad[2];
  const bool inside = i0 >= 0 && i0 < a.in[0] && i1 >= 0 && i1 < a.in[1] && i2 >= 0 && i2 < a.in[2];
  const int64_t src = (((img * a.in[0] + i0) * a.in[1] + i1) * a.in[2] + i2) * a.c + ch;
  uint8_t* dst = a.out + row * a.k + kp;
  if constexpr (VEC == 16) {
    uint4 v = make_uint4(0u, 0u, 0u, 0u);
    if (inside) v = *reinterpret_cast<const uint4*>(a.x + src);
    *reinterpret_cast<uint4*>(dst) = v;
  } else {
    *dst = inside ? a.x[src] : (uint8_t)0;
  }
}

}  // namespace
}  // namespace aqtx

using namespace aqtx;

extern "C" int aqtx_im2col_i8(const aqtx_im2col_plan* p, const void* x, void* out, void* stream) {
  clear_error();
  AQTX_REQUIRE(p != nullptr, "aqtx_im2col_i8: plan is NULL");
  AQTX_REQUIRE(p->rank >= 1 && p->rank <= 3, "aqtx_im2col_i8: spatial rank %d outside 1..3", p->rank);
  AQTX_REQUIRE(p->n >= 0 && p->c >= 0, "aqtx_im2col_i8: negative shape");
  Im2colArgs a{};
  int64_t positions = 1, taps = 1, in_elems = 1;
  for (int d = 0; d < 3; ++d) {
    const int s = d - (3 - p->rank);  // missing leading axes have extent 1
    a.in[d] = s < 0 ? 1 : p->in_size[s];
    a.ker[d] = s < 0 ? 1 : p->kernel[s];
    a.str[d] = s < 0 ? 1 : p->stride[s];
    a.dil[d] = s < 0 ? 1 : p->dilation[s];
    a.pad[d] = s < 0 ? 0 : p->pad_lo[s];
    a.osz[d] = s < 0 ? 1 : p->out_size[s];
    AQTX_REQUIRE(a.in[d] >= 0 && a.ker[d] >= 1 && a.str[d] >= 1 && a.dil[d] >= 1 && a.pad[d] >= 0 && a.osz[d] >= 0,
                 "aqtx_im2col_i8: bad extent on spatial axis %d", s);
    // the last window must start inside the padded input: nothing past pad_lo + in + pad_hi is read,
    // and whatever lies outside [0, in) reads as zero
    positions *= a.osz[d];
    taps *= a.ker[d];
    in_elems *= a.in[d];
  }
  a.rows = p->n * positions;
  a.k = taps * p->c;
  a.c = p->c;
  if (a.rows == 0 || a.k == 0) return 0;
  AQTX_REQUIRE(x != nullptr && out != nullptr, "aqtx_im2col_i8: NULL buffer");
  AQTX_REQUIRE(p->n * in_elems * p->c < (1ll << 40) && a.rows * a.k < (1ll << 40), "aqtx_im2col_i8: tensor too large");
  a.x = reinterpret_cast<const uint8_t*>(x);
  a.out = reinterpret_cast<uint8_t*>(out);
  const bool vec = (p->c % 16) == 0 && ((uintptr_t)x % 16) == 0 && ((uintptr_t)out % 16) == 0;
  const int64_t work = a.rows * (vec ? a.k / 16 : a.k);
  const int64_t blocks = (work + 255) / 256;
  AQTX_REQUIRE(blocks < (1ll << 31), "aqtx_im2col_i8: too many elements for one launch");
  hipStream_t st = reinterpret_cast<hipStream_t>(stream);
  if (vec) im2col_kernel<16><<<(unsigned)blocks, 256, 0, st>>>(a);
  else im2col_kernel<1><<<(unsigned)blocks, 256, 0, st>>>(a);
  AQTX_HIP_CHECK_LAUNCH("im2col_kernel");
  return 0;
}

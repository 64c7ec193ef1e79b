// Two-input elementwise ops with broadcasting on int8 channels-last tensors:
// EltwiseMax / Min / Mul (core/eltwise.cpp:143-347) and BroadcastAdd / Mul / Sub
// (core/broadcast.cpp:45-154).  One lane = 16 channels of one output pixel; an
// operand dimension of 1 repeats along that dimension (a channel count of 1 repeats
// one byte over the 16 lanes of the group).
#include "common.hpp"

using namespace tpuhip;

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;

struct BinArgs {
  const int8_t *x0, *x1;
  int8_t *y;
  int op;
  int n, h, w, c, cs;
  int n0, h0, w0, c0, cs0;
  int n1, h1, w1, c1, cs1;
  int m0, m1, rshift, relu;
  int32_t qmult;   // mul: the qdm multiplier
  int64_t total;   // output pixels * 16-channel groups
};

__device__ __forceinline__ int32_t sb(int32_t word, int i) { return (int32_t)(int8_t)(word >> (8 * i)); }

__device__ __forceinline__ v4i load_operand(const int8_t *x, int pix, int cs, int c, int cg) {
  if (c == 1) {
    const int32_t s = (int32_t)((uint32_t)(uint8_t)x[(int64_t)pix * cs] * 0x01010101u);
    return v4i{s, s, s, s};
  }
  return *reinterpret_cast<const v4i *>(x + (int64_t)pix * cs + cg * 16);
}

// PIXELWISE: neither operand repeats along n, h or w, so both read the output's pixel and
// the index arithmetic below disappears (a channel count of 1 may still repeat).
template <bool PIXELWISE>
__global__ __launch_bounds__(kThreads) void binary_kernel(BinArgs a) {
  const int c16 = a.cs >> 4;
  const int32_t rnd = a.rshift > 0 ? (1 << (a.rshift - 1)) : 0;
  const int32_t mask = (int32_t)((1u << a.rshift) - 1u);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % c16);
    const int pix = (int)(i / c16);
    int p0 = pix, p1 = pix;
    if (!PIXELWISE) {
      const int w = pix % a.w;
      const int h = (pix / a.w) % a.h;
      const int n = pix / (a.w * a.h);
      p0 = ((a.n0 == 1 ? 0 : n) * a.h0 + (a.h0 == 1 ? 0 : h)) * a.w0 + (a.w0 == 1 ? 0 : w);
      p1 = ((a.n1 == 1 ? 0 : n) * a.h1 + (a.h1 == 1 ? 0 : h)) * a.w1 + (a.w1 == 1 ? 0 : w);
    }
    const v4i v0 = load_operand(a.x0, p0, a.cs0, a.c0, cg);
    const v4i v1 = load_operand(a.x1, p1, a.cs1, a.c1, cg);
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int32_t x = sb(v0[q], b), y = sb(v1[q], b);
        int32_t r;
        if (a.op == TPUHIP_BIN_MUL) {
          int32_t v = x * y;
          if (a.relu) v = max(v, 0);
          r = requant_qdm(v, a.qmult, a.rshift, mask, mask >> 1, -128);
        } else {
          const int32_t s = x * a.m0, t = y * a.m1;
          int32_t v = a.op == TPUHIP_BIN_ADD ? s + t
                      : a.op == TPUHIP_BIN_SUB ? s - t
                      : a.op == TPUHIP_BIN_MAX ? max(s, t) : min(s, t);
          if (a.relu) v = max(v, 0);
          r = clamp_i32((v + rnd) >> a.rshift, -128, 127);
        }
        if (cg * 16 + q * 4 + b >= a.c) r = 0;   // pad channels stay zero
        word |= ((uint32_t)r & 0xffu) << (8 * b);
      }
      out[q] = (int)word;
    }
    *reinterpret_cast<v4i *>(a.y + (int64_t)pix * a.cs + cg * 16) = out;
  }
}

}  // namespace

extern "C" int tpuhip_binary_i8(tpuhip_ctx *ctx, const tpuhip_binary_desc *d, const void *x0,
                                const void *x1, void *y) {
  TPUHIP_REQUIRE(ctx && d && x0 && x1 && y, "binary: NULL argument");
  TPUHIP_REQUIRE(d->op >= TPUHIP_BIN_ADD && d->op <= TPUHIP_BIN_MUL, "binary: unknown op %d", d->op);
  TPUHIP_REQUIRE(d->n > 0 && d->c > 0 && d->h > 0 && d->w > 0, "binary: non-positive dimension");
  const int dims[2][4] = {{d->n0, d->c0, d->h0, d->w0}, {d->n1, d->c1, d->h1, d->w1}};
  const int out[4] = {d->n, d->c, d->h, d->w};
  for (int k = 0; k < 2; ++k)
    for (int j = 0; j < 4; ++j)
      TPUHIP_REQUIRE(dims[k][j] == out[j] || dims[k][j] == 1,
                     "binary: operand %d dimension %d is %d, neither 1 nor the output's %d", k, j,
                     dims[k][j], out[j]);
  TPUHIP_REQUIRE(d->y_cs >= d->c && d->y_cs % 16 == 0 && d->x0_cs >= d->c0 && d->x0_cs % 16 == 0 &&
                     d->x1_cs >= d->c1 && d->x1_cs % 16 == 0,
                 "binary: channel strides must be multiples of 16 covering the channels");
  TPUHIP_REQUIRE(d->c0 == 1 || d->x0_cs == d->y_cs, "binary: operand 0 channel stride differs from the output's");
  TPUHIP_REQUIRE(d->c1 == 1 || d->x1_cs == d->y_cs, "binary: operand 1 channel stride differs from the output's");
  TPUHIP_REQUIRE(d->rshift >= 0 && d->rshift <= 31, "binary: rshift %d outside [0,31]", d->rshift);
  if (d->op == TPUHIP_BIN_MUL) {
    TPUHIP_REQUIRE(d->rshift != 0 || d->multiplier != 0,
                   "binary: a product with rshift 0 and multiplier 0 has no int8 meaning "
                   "(the reference keeps the raw product)");
  } else {
    TPUHIP_REQUIRE(d->rshift <= 30, "binary: rshift %d outside [0,30]", d->rshift);
    TPUHIP_REQUIRE(d->m0 >= -128 && d->m0 <= 127 && d->m1 >= -128 && d->m1 <= 127,
                   "binary: multipliers must be int8");
  }
  TPUHIP_REQUIRE((int64_t)d->n * d->h * d->w < (1ll << 31), "binary: tensor too large");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  BinArgs a{};
  a.x0 = (const int8_t *)x0; a.x1 = (const int8_t *)x1; a.y = (int8_t *)y;
  a.op = d->op;
  a.n = d->n; a.h = d->h; a.w = d->w; a.c = d->c; a.cs = d->y_cs;
  a.n0 = d->n0; a.h0 = d->h0; a.w0 = d->w0; a.c0 = d->c0; a.cs0 = d->x0_cs;
  a.n1 = d->n1; a.h1 = d->h1; a.w1 = d->w1; a.c1 = d->c1; a.cs1 = d->x1_cs;
  a.m0 = d->m0; a.m1 = d->m1; a.rshift = d->rshift; a.relu = d->do_relu ? 1 : 0;
  a.qmult = d->multiplier;
  a.total = (int64_t)d->n * d->h * d->w * (d->y_cs / 16);
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(a.total, kThreads), (int64_t)ctx->num_cu * 32));
  const bool pixelwise = d->n0 == d->n && d->h0 == d->h && d->w0 == d->w && d->n1 == d->n &&
                         d->h1 == d->h && d->w1 == d->w;
  if (pixelwise)
    launch(ctx, binary_kernel<true>, dim3(blocks), dim3(kThreads), a);
  else
    launch(ctx, binary_kernel<false>, dim3(blocks), dim3(kThreads), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

// INT8 max / average pooling for gfx950, channels-last: one lane owns 16
// channels of one output pixel (16-byte loads and stores).  Bandwidth-bound,
// no MFMA.
#include "common.hpp"

#include <algorithm>

using namespace tpuhip;

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

struct PoolArgs {
  const int8_t *x;
  int8_t *y;
  int n, c16, ih, iw, oh, ow, kh, kw, sh, sw, pt, pl, x_cs, y_cs;
  float mult;       // (float)multiplier
  float inv_pot;    // 2^-rshift
};

__device__ __forceinline__ int32_t sb(int32_t word, int i) {
  return (int32_t)(int8_t)(word >> (8 * i));
}

// Workgroups are dealt to the 8 XCDs round-robin.  With a grid that is a multiple of 8 this
// renumbering gives every XCD a contiguous run of logical blocks, i.e. of output rows, so the
// input rows that neighbouring windows share are fetched into one L2 instead of several.
__device__ __forceinline__ unsigned xcd_block() {
  return (blockIdx.x & 7u) * (gridDim.x >> 3) + (blockIdx.x >> 3);
}

// PoolingOpKernel INT8 max (core/pooling.cpp:155-157): MKL-DNN pooling_max skips
// padded positions.
__global__ __launch_bounds__(256) void pool_max_kernel(PoolArgs a) {
  const int64_t total = (int64_t)a.n * a.oh * a.ow * a.c16;
  for (int64_t i = (int64_t)xcd_block() * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % a.c16);
    int64_t p = i / a.c16;
    const int ow = (int)(p % a.ow);
    p /= a.ow;
    const int oh = (int)(p % a.oh);
    const int b = (int)(p / a.oh);
    int32_t best[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) best[k] = -128;
    for (int kh = 0; kh < a.kh; ++kh) {
      const int ih = oh * a.sh - a.pt + kh;
      if (ih < 0 || ih >= a.ih) continue;
      for (int kw = 0; kw < a.kw; ++kw) {
        const int iw = ow * a.sw - a.pl + kw;
        if (iw < 0 || iw >= a.iw) continue;
        const v4i v = *reinterpret_cast<const v4i *>(
            a.x + ((int64_t)(b * a.ih + ih) * a.iw + iw) * a.x_cs + cg * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int k = 0; k < 4; ++k) best[q * 4 + k] = max(best[q * 4 + k], sb(v[q], k));
      }
    }
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t w = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) w |= ((uint32_t)best[q * 4 + k] & 0xffu) << (8 * k);
      out[q] = (int)w;
    }
    *reinterpret_cast<v4i *>(a.y + ((int64_t)(b * a.oh + oh) * a.ow + ow) * a.y_cs + cg * 16) = out;
  }
}

// PoolingOpKernel INT8 average, normal path (core/pooling.cpp:147-154): window
// sum with zero padding, then the float overload of
// applyMultiplierAndRShiftAndSaturateInt8 without qdm: float product, float
// quotient by a power of two, floor(f + 0.5), clamp.
__global__ __launch_bounds__(256) void pool_avg_kernel(PoolArgs a) {
  const int64_t total = (int64_t)a.n * a.oh * a.ow * a.c16;
  for (int64_t i = (int64_t)xcd_block() * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % a.c16);
    int64_t p = i / a.c16;
    const int ow = (int)(p % a.ow);
    p /= a.ow;
    const int oh = (int)(p % a.oh);
    const int b = (int)(p / a.oh);
    int32_t sum[16];
#pragma unroll
    for (int k = 0; k < 16; ++k) sum[k] = 0;
    for (int kh = 0; kh < a.kh; ++kh) {
      const int ih = oh * a.sh - a.pt + kh;
      if (ih < 0 || ih >= a.ih) continue;
      for (int kw = 0; kw < a.kw; ++kw) {
        const int iw = ow * a.sw - a.pl + kw;
        if (iw < 0 || iw >= a.iw) continue;
        const v4i v = *reinterpret_cast<const v4i *>(
            a.x + ((int64_t)(b * a.ih + ih) * a.iw + iw) * a.x_cs + cg * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int k = 0; k < 4; ++k) sum[q * 4 + k] += sb(v[q], k);
      }
    }
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t w = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float prod = __fmul_rn((float)sum[q * 4 + k], a.mult);
        const float quo = __fmul_rn(prod, a.inv_pot);  // exact: power-of-two scaling
        w |= ((uint32_t)saturate_int8_f(quo) & 0xffu) << (8 * k);
      }
      out[q] = (int)w;
    }
    *reinterpret_cast<v4i *>(a.y + ((int64_t)(b * a.oh + oh) * a.ow + ow) * a.y_cs + cg * 16) = out;
  }
}

// Global / large-window average pooling: LANES lanes share one (pixel, 16-channel
// group) output, each sums every LANES-th window position, and the partial sums
// meet through wave shuffles.  Keeps enough loads in flight when there are few
// outputs (a 7x7 global pool has 49 taps per output and only n*c/16 outputs).
template <int LANES>
__global__ __launch_bounds__(256) void pool_avg_split_kernel(PoolArgs a) {
  const int64_t total = (int64_t)a.n * a.oh * a.ow * a.c16;
  const int64_t gid = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) / LANES;
  const int sub = threadIdx.x % LANES;
  const bool live = gid < total;
  const int64_t i = live ? gid : 0;
  const int cg = (int)(i % a.c16);
  int64_t p = i / a.c16;
  const int ow = (int)(p % a.ow);
  p /= a.ow;
  const int oh = (int)(p % a.oh);
  const int b = (int)(p / a.oh);
  int32_t sum[16];
#pragma unroll
  for (int k = 0; k < 16; ++k) sum[k] = 0;
  const int taps = a.kh * a.kw;
  // up to MAXT window positions of this lane are requested before any is added, so their
  // latencies overlap instead of lining up one behind the other
  constexpr int MAXT = 8;
  const uint32_t magic_kw = (1u << 20) / (uint32_t)a.kw + 1;   // t / kw == (t * magic) >> 20 for t < 4095
  for (int t0 = sub; t0 < taps; t0 += LANES * MAXT) {
    v4i v[MAXT];
#pragma unroll
    for (int u = 0; u < MAXT; ++u) {
      const int t = t0 + u * LANES;
      const int kh = (int)(((uint32_t)t * magic_kw) >> 20), kw = t - kh * a.kw;
      const int ih = oh * a.sh - a.pt + kh, iw = ow * a.sw - a.pl + kw;
      const bool ok = (t < taps) & ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
      v[u] = v4i{0, 0, 0, 0};
      if (ok)
        v[u] = *reinterpret_cast<const v4i *>(a.x + ((int64_t)(b * a.ih + ih) * a.iw + iw) * a.x_cs + cg * 16);
    }
#pragma unroll
    for (int u = 0; u < MAXT; ++u)
#pragma unroll
      for (int q = 0; q < 4; ++q)
#pragma unroll
        for (int k = 0; k < 4; ++k) sum[q * 4 + k] += sb(v[u][q], k);
  }
#pragma unroll
  for (int k = 0; k < 16; ++k)
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) sum[k] += __shfl_xor(sum[k], off, LANES);
  if (live && sub == 0) {
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t w = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float prod = __fmul_rn((float)sum[q * 4 + k], a.mult);
        const float quo = __fmul_rn(prod, a.inv_pot);
        w |= ((uint32_t)saturate_int8_f(quo) & 0xffu) << (8 * k);
      }
      out[q] = (int)w;
    }
    *reinterpret_cast<v4i *>(a.y + ((int64_t)(b * a.oh + oh) * a.ow + ow) * a.y_cs + cg * 16) = out;
  }
}

int fill_args(const tpuhip_pool_desc *d, const void *x, void *y, PoolArgs *a) {
  TPUHIP_REQUIRE(d && x && y, "pool: NULL argument");
  TPUHIP_REQUIRE(d->n > 0 && d->c > 0 && d->ih > 0 && d->iw > 0 && d->oh > 0 && d->ow > 0 &&
                     d->kh > 0 && d->kw > 0 && d->sh > 0 && d->sw > 0,
                 "pool: non-positive dimension");
  TPUHIP_REQUIRE(d->pt >= 0 && d->pb >= 0 && d->pl >= 0 && d->pr >= 0, "pool: negative padding");
  TPUHIP_REQUIRE(d->x_cs % 16 == 0 && d->y_cs % 16 == 0 && d->x_cs >= d->c && d->y_cs >= d->c,
                 "pool: bad channel strides %d / %d for %d channels", d->x_cs, d->y_cs, d->c);
  // every window must contain at least one real input position
  TPUHIP_REQUIRE((d->oh - 1) * d->sh - d->pt < d->ih && (d->ow - 1) * d->sw - d->pl < d->iw &&
                     d->pt < d->kh && d->pl < d->kw,
                 "pool: an output window lies entirely in the padding");
  a->x = (const int8_t *)x;
  a->y = (int8_t *)y;
  a->n = d->n; a->c16 = (d->c + 15) / 16;
  a->ih = d->ih; a->iw = d->iw; a->oh = d->oh; a->ow = d->ow;
  a->kh = d->kh; a->kw = d->kw; a->sh = d->sh; a->sw = d->sw;
  a->pt = d->pt; a->pl = d->pl; a->x_cs = d->x_cs; a->y_cs = d->y_cs;
  a->mult = 0.f; a->inv_pot = 1.f;
  return TPUHIP_OK;
}

unsigned blocks_for(const PoolArgs &a) {
  const int64_t total = (int64_t)a.n * a.oh * a.ow * a.c16;
  // a multiple of 8 (see xcd_block)
  return 8u * (unsigned)std::max<int64_t>(1, std::min<int64_t>((total + 2047) / 2048, 1 << 13));
}

}  // namespace

extern "C" {

int tpuhip_pool_max_i8(tpuhip_ctx *ctx, const tpuhip_pool_desc *d, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx, "pool_max: NULL context");
  PoolArgs a;
  if (int rc = fill_args(d, x, y, &a)) return rc;
  launch(ctx, pool_max_kernel, dim3(blocks_for(a)), dim3(256), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_pool_avg_i8(tpuhip_ctx *ctx, const tpuhip_pool_desc *d, const void *x, void *y,
                       uint32_t multiplier, uint32_t rshift) {
  TPUHIP_REQUIRE(ctx, "pool_avg: NULL context");
  TPUHIP_REQUIRE(rshift <= 30, "pool_avg: rshift %u outside [0,30]", rshift);
  PoolArgs a;
  if (int rc = fill_args(d, x, y, &a)) return rc;
  TPUHIP_REQUIRE((int64_t)d->kh * d->kw * 128 < (1 << 24), "pool_avg: window too large");
  a.mult = (float)multiplier;
  a.inv_pot = 1.0f / (float)(1 << rshift);
  const int64_t outputs = (int64_t)a.n * a.oh * a.ow * a.c16;
  if (d->kh * d->kw >= 16 && outputs < (1 << 16)) {
    const unsigned blocks = (unsigned)((outputs * 8 + 255) / 256);
    launch(ctx, pool_avg_split_kernel<8>, dim3(blocks), dim3(256), a);
  } else {
    launch(ctx, pool_avg_kernel, dim3(blocks_for(a)), dim3(256), a);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // extern "C"

// Bandwidth-bound INT8 ops for gfx950: eltwise add, 256-entry table ops
// (leaky-ReLU / clip / LUT activations), ReLU, nearest upsample, concat and the
// NCHW <-> channels-last conversions at the API edge.  All kernels move 16
// bytes per lane per access where the layout allows it; none uses MFMA.
#include "common.hpp"

#include <cstring>

#include <algorithm>
#include <cmath>

using namespace tpuhip;

typedef int v4i __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256;

inline unsigned grid_for(int64_t items, int per_block = kThreads, int64_t cap = 1 << 16) {
  return (unsigned)std::max<int64_t>(1, std::min<int64_t>(ceil_div64(items, per_block), cap));
}

__device__ __forceinline__ int32_t sb(int32_t word, int i) {
  return (int32_t)(int8_t)(word >> (8 * i));
}

// ---------------------------------------------------------------------------
// eltwise add (core/eltwise.cpp:52-85).  The reference forms sum_i x_i * m_i and
// sum / 2^r in float; both are exact for |sum| < 2^24 (at most 8 inputs of
// 128 * 128), so the integer form floor((sum + 2^(r-1)) / 2^r) is identical.
// ---------------------------------------------------------------------------
struct EltArgs {
  const int8_t *x[8];
  int8_t *y;
  int32_t m[8];
  int nin;
  int rshift;
  int relu;
  int64_t n16;   // number of 16-byte groups
};

template <int NIN>
__global__ __launch_bounds__(kThreads) void eltwise_add_kernel(EltArgs a) {
  const int32_t rnd = a.rshift > 0 ? (1 << (a.rshift - 1)) : 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.n16;
       i += (int64_t)gridDim.x * blockDim.x) {
    v4i in[NIN];
#pragma unroll
    for (int k = 0; k < NIN; ++k) in[k] = reinterpret_cast<const v4i *>(a.x[k])[i];
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        int32_t s = 0;
#pragma unroll
        for (int k = 0; k < NIN; ++k) s += sb(in[k][q], b) * a.m[k];
        if (a.relu) s = max(s, 0);
        s = clamp_i32((s + rnd) >> a.rshift, -128, 127);
        word |= ((uint32_t)s & 0xffu) << (8 * b);
      }
      out[q] = (int)word;
    }
    reinterpret_cast<v4i *>(a.y)[i] = out;
  }
}

// ---------------------------------------------------------------------------
// one 256-entry table per channel (PRelu's per-channel slope, core/activation.cpp:185-224):
// y[pixel][c] = tables[c][(unsigned char)x[pixel][c]].  One lane = 16 channels of a pixel;
// the tables (c * 256 bytes) stay in the caches.  Pad channels are written as zero.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void lut_per_channel_kernel(const int8_t *x, int8_t *y,
                                                                   const uint8_t *tables,
                                                                   int64_t total, int c, int cs) {
  const int c16 = cs >> 4;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % c16);
    const v4i in = reinterpret_cast<const v4i *>(x)[i];
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int ch = cg * 16 + q * 4 + b;
        const uint32_t idx = ((uint32_t)in[q] >> (8 * b)) & 255u;
        const uint32_t r = ch < c ? tables[(size_t)ch * 256 + idx] : 0u;
        word |= r << (8 * b);
      }
      out[q] = (int)word;
    }
    reinterpret_cast<v4i *>(y)[i] = out;
  }
}

// ---------------------------------------------------------------------------
// table ops: y = table[(unsigned char)x] (core/activation.cpp:47-53).  The table
// arrives by value in the kernel arguments and is spread into LDS once per
// workgroup; pad channels are forced to zero.
// ---------------------------------------------------------------------------
struct LutArgs {
  const int8_t *x;
  int8_t *y;
  int64_t pixels;
  int c, x_cs, y_cs;  // channels, strides
  int coff;           // channel offset into y (concat)
  int use_table;
};

__device__ __forceinline__ void table_to_lds(const Table256 &t, uint8_t *lds) {
  // every thread writes the same words; constant indexing keeps the table in SGPRs
  uint32_t *l32 = reinterpret_cast<uint32_t *>(lds);
  if (threadIdx.x < 64) {
#pragma unroll
    for (int i = 0; i < 64; ++i)
      if ((int)threadIdx.x == i) l32[i] = t.w[i];
  }
  __syncthreads();
}

// vector form: c16 groups of 16 channels per pixel, strides multiple of 16, coff multiple of 16
__global__ __launch_bounds__(kThreads) void lut_vec_kernel(LutArgs a, Table256 t) {
  __shared__ uint8_t tab[256];
  table_to_lds(t, tab);
  const int c16 = (a.c + 15) >> 4;
  const int64_t total = a.pixels * c16;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t pix = i / c16;
    const int cg = (int)(i - pix * c16);
    v4i v = *reinterpret_cast<const v4i *>(a.x + pix * a.x_cs + cg * 16);
    if (a.use_table) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint32_t w = (uint32_t)v[q], o = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int ch = cg * 16 + q * 4 + b;
          const uint32_t e = ch < a.c ? tab[(w >> (8 * b)) & 0xffu] : 0u;
          o |= e << (8 * b);
        }
        v[q] = (int)o;
      }
    }
    *reinterpret_cast<v4i *>(a.y + pix * a.y_cs + a.coff + cg * 16) = v;
  }
}

// byte form for channel offsets / counts that are not multiples of 16
__global__ __launch_bounds__(kThreads) void lut_byte_kernel(LutArgs a, Table256 t) {
  __shared__ uint8_t tab[256];
  table_to_lds(t, tab);
  const int64_t total = a.pixels * a.c;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t pix = i / a.c;
    const int ch = (int)(i - pix * a.c);
    uint8_t v = (uint8_t)a.x[pix * a.x_cs + ch];
    if (a.use_table) v = tab[v];
    a.y[pix * a.y_cs + a.coff + ch] = (int8_t)v;
  }
}

// concat of up to four inputs that changes no byte, along any axis: in channels-last memory every
// axis is "for each outer index, the inputs' chunks one after the other" (outer = pixel for the
// channel axis, image row for w, image for h, nothing for n), chunks whole 16-byte groups.
// One launch, a lane moves one 16-byte group.
struct ConcatArgs {
  const int8_t *x[4];
  int8_t *y;
  int64_t outer;       // outer indices
  int64_t stride[4];   // bytes from one outer index to the next in each input
  int64_t y_stride;    // ... in the output
  int64_t start[5];    // first 16-byte group of each input's chunk within an output chunk; start[n] = groups per chunk
  int64_t groups;      // groups written per outer index (>= start[n]; the rest are zero)
  int n;
};

__global__ __launch_bounds__(kThreads) void concat_chunks_kernel(ConcatArgs a) {
  const int64_t g16 = a.groups;   // groups written per outer index: those of the inputs, then zero pad groups
  const int64_t total = a.outer * g16;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t o = i / g16;
    const int64_t g = i - o * g16;
    // which input the group comes from: selects, so that no array is indexed by a lane's value
    const int8_t *src = a.x[0];
    int64_t stride = a.stride[0], first = 0;
    if (a.n > 1 && g >= a.start[1]) { src = a.x[1]; stride = a.stride[1]; first = a.start[1]; }
    if (a.n > 2 && g >= a.start[2]) { src = a.x[2]; stride = a.stride[2]; first = a.start[2]; }
    if (a.n > 3 && g >= a.start[3]) { src = a.x[3]; stride = a.stride[3]; first = a.start[3]; }
    v4i v = {0, 0, 0, 0};
    if (g < a.start[a.n]) v = *reinterpret_cast<const v4i *>(src + o * stride + (g - first) * 16);
    *reinterpret_cast<v4i *>(a.y + o * a.y_stride + g * 16) = v;
  }
}

// zero the channels [c0, c1) of every pixel
__global__ __launch_bounds__(kThreads) void zero_channels_kernel(int8_t *y, int64_t pixels, int cs,
                                                                 int c0, int c1) {
  const int w = c1 - c0;
  const int64_t total = pixels * w;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t pix = i / w;
    y[pix * cs + c0 + (int)(i - pix * w)] = 0;
  }
}

__global__ __launch_bounds__(kThreads) void relu_kernel(const v4i *x, v4i *y, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16;
       i += (int64_t)gridDim.x * blockDim.x) {
    v4i v = x[i];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t w = (uint32_t)v[q];
      // a byte with its sign bit set becomes 0
      uint32_t neg = (w & 0x80808080u) >> 7;   // 1 per negative byte
      uint32_t mask = neg * 0xffu;             // 0xff per negative byte
      v[q] = (int)(w & ~mask);
    }
    y[i] = v;
  }
}

// ---------------------------------------------------------------------------
// nearest upsample (core/upsample.cpp:20-41), channels-last: one 16-byte group
// of an output pixel per lane.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void upsample_kernel(const int8_t *x, int8_t *y, int n,
                                                            int ih, int iw, int sh, int sw,
                                                            int c16, int x_cs, int y_cs) {
  const int oh = ih * sh, ow = iw * sw;
  const int64_t total = (int64_t)n * oh * ow * c16;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % c16);
    int64_t p = i / c16;
    const int wo = (int)(p % ow);
    p /= ow;
    const int ho = (int)(p % oh);
    const int b = (int)(p / oh);
    const int64_t src = ((int64_t)(b * ih + ho / sh) * iw + wo / sw) * x_cs + cg * 16;
    const int64_t dst = ((int64_t)(b * oh + ho) * ow + wo) * y_cs + cg * 16;
    *reinterpret_cast<v4i *>(y + dst) = *reinterpret_cast<const v4i *>(x + src);
  }
}

// ---------------------------------------------------------------------------
// layout conversion through an LDS tile: reads are contiguous along W (NCHW
// side), writes contiguous along C (channels-last side) and vice versa.
// ---------------------------------------------------------------------------
template <typename SRC>
__global__ __launch_bounds__(kThreads) void nchw_to_nhwc_kernel(const SRC *src, int8_t *dst, int c,
                                                                int64_t hw, int cs) {
  // block: 64 spatial positions x 64 channels of one image
  __shared__ int8_t tile[64][65];
  const int n = blockIdx.z;
  const int64_t s0 = (int64_t)blockIdx.x * 64;
  const int c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;  // 4 rows of 64
  for (int r = ty; r < 64; r += 4) {
    const int ch = c0 + r;
    const int64_t s = s0 + tx;
    int8_t v = 0;
    if (ch < c && s < hw) v = (int8_t)src[((int64_t)n * c + ch) * hw + s];
    tile[r][tx] = v;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int64_t s = s0 + r;
    const int ch = c0 + tx;
    if (s < hw && ch < cs) dst[((int64_t)n * hw + s) * cs + ch] = tile[tx][r];
  }
}

template <typename DST>
__global__ __launch_bounds__(kThreads) void nhwc_to_nchw_kernel(const int8_t *src, DST *dst, int c,
                                                                int64_t hw, int cs) {
  __shared__ int8_t tile[64][65];
  const int n = blockIdx.z;
  const int64_t s0 = (int64_t)blockIdx.x * 64;
  const int c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  for (int r = ty; r < 64; r += 4) {
    const int64_t s = s0 + r;
    const int ch = c0 + tx;
    int8_t v = 0;
    if (s < hw && ch < c) v = src[((int64_t)n * hw + s) * cs + ch];
    tile[r][tx] = v;
  }
  __syncthreads();
  for (int r = ty; r < 64; r += 4) {
    const int ch = c0 + r;
    const int64_t s = s0 + tx;
    if (ch < c && s < hw) dst[((int64_t)n * c + ch) * hw + s] = (DST)tile[tx][r];
  }
}

int check_layout_args(const void *a, const void *b, int n, int c, int h, int w, int cs) {
  TPUHIP_REQUIRE(a && b, "layout: NULL pointer");
  TPUHIP_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0, "layout: non-positive dimension");
  TPUHIP_REQUIRE(cs >= c && (cs % 16 == 0 || cs == 4), "layout: channel stride %d must be 4 or a multiple of 16, >= %d",
                 cs, c);
  TPUHIP_REQUIRE(n <= 65535 && (c + 63) / 64 <= 65535, "layout: too many images / channels");
  return TPUHIP_OK;
}

template <typename SRC>
int to_nhwc(tpuhip_ctx *ctx, const void *src, void *dst, int n, int c, int h, int w, int cs) {
  TPUHIP_REQUIRE(ctx, "layout: NULL context");
  if (int rc = check_layout_args(src, dst, n, c, h, w, cs)) return rc;
  const int64_t hw = (int64_t)h * w;
  dim3 grid((unsigned)ceil_div64(hw, 64), (unsigned)((cs + 63) / 64), (unsigned)n);
  launch(ctx, (nchw_to_nhwc_kernel<SRC>), grid, dim3(kThreads), (const SRC *)src, (int8_t *)dst, c, hw, cs);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

template <typename DST>
int to_nchw(tpuhip_ctx *ctx, const void *src, void *dst, int n, int c, int h, int w, int cs) {
  TPUHIP_REQUIRE(ctx, "layout: NULL context");
  if (int rc = check_layout_args(src, dst, n, c, h, w, cs)) return rc;
  const int64_t hw = (int64_t)h * w;
  dim3 grid((unsigned)ceil_div64(hw, 64), (unsigned)((c + 63) / 64), (unsigned)n);
  launch(ctx, (nhwc_to_nchw_kernel<DST>), grid, dim3(kThreads), (const int8_t *)src, (DST *)dst, c, hw, cs);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

// host: saturateInt8 of v * multiplier / 2^rshift evaluated in float32 the way
// applyMultiplierAndRShiftAndSaturateInt8's float overload does
// (QuantizationArithmetic.cpp:518-528, :301-334)
int8_t host_mult_rshift_sat8(float v, uint32_t rshift, uint32_t multiplier) {
  volatile float prod = v * (float)multiplier;
  volatile float quo = prod / (float)(1 << rshift);
  double s = std::floor((double)quo + 0.5);
  if (s > 127.0) s = 127.0;
  if (s < -128.0) s = -128.0;
  return (int8_t)(int)s;
}

Table256 pack_table(const int8_t *t) {
  Table256 r;
  for (int i = 0; i < 64; ++i)
    r.w[i] = (uint32_t)(uint8_t)t[4 * i] | ((uint32_t)(uint8_t)t[4 * i + 1] << 8) |
             ((uint32_t)(uint8_t)t[4 * i + 2] << 16) | ((uint32_t)(uint8_t)t[4 * i + 3] << 24);
  return r;
}

int launch_lut(tpuhip_ctx *ctx, const void *x, void *y, const int8_t *table, int64_t pixels, int c,
               int x_cs, int y_cs, int coff) {
  LutArgs a{};
  a.x = (const int8_t *)x;
  a.y = (int8_t *)y;
  a.pixels = pixels;
  a.c = c;
  a.x_cs = x_cs;
  a.y_cs = y_cs;
  a.coff = coff;
  a.use_table = table != nullptr;
  Table256 t{};
  if (table) t = pack_table(table);
  const bool vec = (x_cs % 16 == 0) && (y_cs % 16 == 0) && (coff % 16 == 0) &&
                   (c % 16 == 0 || (coff + round_up(c, 16) <= y_cs));
  if (vec) {
    const int64_t total = pixels * ((c + 15) / 16);
    launch(ctx, lut_vec_kernel, dim3(grid_for(total, kThreads * 4)), dim3(kThreads), a, t);
  } else {
    launch(ctx, lut_byte_kernel, dim3(grid_for(pixels * c, kThreads * 8)), dim3(kThreads), a, t);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

// INT8 LRN across channels (core/lrn.cpp:104-166).  A lane produces four consecutive channels
// of a pixel; the window of local_size channels around each is summed from the squares table
// (indexed by the input byte), rescaled to an index into the power table, and that entry
// scales the input.  All integers: the reference's float arithmetic is exact for them.
struct LrnArgs {
  const int8_t *x;
  int8_t *y;
  int64_t total;   // pixels * (cs / 4)
  int c, cs, local_size, sum_rshift, lrn_rshift, quant0, quant1;
  Table256 sqr, power;
};

__global__ __launch_bounds__(kThreads) void lrn_kernel(LrnArgs a) {
  __shared__ uint32_t tsq[64], tpw[64];
  if (threadIdx.x < 64) {
    tsq[threadIdx.x] = a.sqr.w[threadIdx.x];
    tpw[threadIdx.x] = a.power.w[threadIdx.x];
  }
  __syncthreads();
  const uint8_t *sq = reinterpret_cast<const uint8_t *>(tsq);
  const uint8_t *pw = reinterpret_cast<const uint8_t *>(tpw);
  const int c4 = a.cs >> 2, pre_pad = (a.local_size - 1) / 2;
  const int rnd_s = a.sum_rshift > 0 ? 1 << (a.sum_rshift - 1) : 0;
  const int rnd_l = a.lrn_rshift > 0 ? 1 << (a.lrn_rshift - 1) : 0;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cq = (int)(i % c4);
    const int64_t pix = i / c4;
    const int8_t *row = a.x + pix * a.cs;
    uint32_t word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int ch = cq * 4 + b;
      if (ch >= a.c) continue;   // pad channels stay zero
      int s = 0;
      const int lo = max(ch - pre_pad, 0), hi = min(ch - pre_pad + a.local_size, a.c);
      for (int k = lo; k < hi; ++k) s += sq[(uint8_t)row[k]];
      const int t = min(max((s * a.quant0 + rnd_s) >> a.sum_rshift, 0), 255);
      const int m = (int)pw[t] * (int)row[ch] * a.quant1;
      const int o = min(max((m + rnd_l) >> a.lrn_rshift, -128), 127);
      word |= (uint32_t)(uint8_t)(int8_t)o << (8 * b);
    }
    *reinterpret_cast<uint32_t *>(a.y + pix * a.cs + cq * 4) = word;
  }
}

}  // namespace

extern "C" {

int tpuhip_nchw_to_nhwc_i8(tpuhip_ctx *ctx, const void *s, void *d, int n, int c, int h, int w,
                           int cs) {
  return to_nhwc<int8_t>(ctx, s, d, n, c, h, w, cs);
}
int tpuhip_nchw_f32_to_nhwc_i8(tpuhip_ctx *ctx, const void *s, void *d, int n, int c, int h, int w,
                               int cs) {
  return to_nhwc<float>(ctx, s, d, n, c, h, w, cs);
}
int tpuhip_nhwc_to_nchw_i8(tpuhip_ctx *ctx, const void *s, void *d, int n, int c, int h, int w,
                           int cs) {
  return to_nchw<int8_t>(ctx, s, d, n, c, h, w, cs);
}
int tpuhip_nhwc_i8_to_nchw_f32(tpuhip_ctx *ctx, const void *s, void *d, int n, int c, int h, int w,
                               int cs) {
  return to_nchw<float>(ctx, s, d, n, c, h, w, cs);
}

int tpuhip_eltwise_add_i8(tpuhip_ctx *ctx, const void *const *xs, int nin,
                          const int8_t *multiplier, int rshift, int do_relu, void *y,
                          size_t bytes) {
  TPUHIP_REQUIRE(ctx && xs && multiplier && y, "eltwise_add: NULL argument");
  TPUHIP_REQUIRE(nin >= 1 && nin <= 8, "eltwise_add: %d inputs (1..8 supported)", nin);
  TPUHIP_REQUIRE(rshift >= 0 && rshift <= 30, "eltwise_add: rshift %d outside [0,30]", rshift);
  TPUHIP_REQUIRE(bytes % 16 == 0, "eltwise_add: byte count %zu not a multiple of 16", bytes);
  if (bytes == 0) return TPUHIP_OK;
  EltArgs a{};
  for (int i = 0; i < nin; ++i) {
    TPUHIP_REQUIRE(xs[i], "eltwise_add: input %d is NULL", i);
    a.x[i] = (const int8_t *)xs[i];
    a.m[i] = multiplier[i];
  }
  a.y = (int8_t *)y;
  a.nin = nin;
  a.rshift = rshift;
  a.relu = do_relu ? 1 : 0;
  a.n16 = (int64_t)(bytes / 16);
  const dim3 grid(grid_for(a.n16, kThreads * 2)), block(kThreads);
  switch (nin) {
    case 1: launch(ctx, eltwise_add_kernel<1>, grid, block, a); break;
    case 2: launch(ctx, eltwise_add_kernel<2>, grid, block, a); break;
    case 3: launch(ctx, eltwise_add_kernel<3>, grid, block, a); break;
    case 4: launch(ctx, eltwise_add_kernel<4>, grid, block, a); break;
    case 5: launch(ctx, eltwise_add_kernel<5>, grid, block, a); break;
    case 6: launch(ctx, eltwise_add_kernel<6>, grid, block, a); break;
    case 7: launch(ctx, eltwise_add_kernel<7>, grid, block, a); break;
    default: launch(ctx, eltwise_add_kernel<8>, grid, block, a); break;
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_lut_i8(tpuhip_ctx *ctx, const void *x, void *y, const int8_t *table256, size_t pixels,
                  int c, int cs) {
  TPUHIP_REQUIRE(ctx && x && y && table256, "lut: NULL argument");
  TPUHIP_REQUIRE(c > 0 && cs >= c && cs % 16 == 0, "lut: bad channels %d / stride %d", c, cs);
  if (pixels == 0) return TPUHIP_OK;
  return launch_lut(ctx, x, y, table256, (int64_t)pixels, c, cs, cs, 0);
}

int tpuhip_lrn_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t pixels, int c, int cs, int local_size,
                  const uint8_t *sqr_lut256, const uint8_t *power_lut256, int sum_rshift, int lrn_rshift,
                  int quant0, int quant1) {
  TPUHIP_REQUIRE(ctx && x && y && sqr_lut256 && power_lut256, "lrn: NULL argument");
  TPUHIP_REQUIRE(c > 0 && cs >= c && cs % 16 == 0, "lrn: bad channels %d / stride %d", c, cs);
  TPUHIP_REQUIRE(local_size >= 1 && local_size <= 64, "lrn: local_size %d outside [1,64]", local_size);
  TPUHIP_REQUIRE(sum_rshift >= 0 && sum_rshift <= 23 && lrn_rshift >= 0 && lrn_rshift <= 23,
                 "lrn: shifts %d / %d outside [0,23]", sum_rshift, lrn_rshift);
  // the reference computes in float; these bounds keep every intermediate an exact integer
  // multiple of a power of two below 2^24, so the integer form used here gives the same bytes
  // (the running sum holds one more term than the window while the head is added before the
  // tail is subtracted; the rounding term is half a unit of the shifted result)
  TPUHIP_REQUIRE(quant0 >= 0 && (int64_t)255 * quant0 * (local_size + 1) + (1ll << sum_rshift) < (1 << 24),
                 "lrn: quant_data0 %d too large for exact float sums", quant0);
  TPUHIP_REQUIRE(quant1 >= 0 && (int64_t)255 * 128 * quant1 + (1ll << lrn_rshift) < (1 << 24),
                 "lrn: quant_data1 %d too large for exact float products", quant1);
  if (pixels == 0) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  LrnArgs a{};
  a.x = (const int8_t *)x;
  a.y = (int8_t *)y;
  a.total = (int64_t)pixels * (cs / 4);
  a.c = c; a.cs = cs; a.local_size = local_size;
  a.sum_rshift = sum_rshift; a.lrn_rshift = lrn_rshift; a.quant0 = quant0; a.quant1 = quant1;
  memcpy(a.sqr.w, sqr_lut256, 256);
  memcpy(a.power.w, power_lut256, 256);
  launch(ctx, lrn_kernel, dim3(grid_for(a.total, kThreads * 2)), dim3(kThreads), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_lut_per_channel_i8(tpuhip_ctx *ctx, const void *x, void *y, const void *tables,
                              size_t pixels, int c, int cs) {
  TPUHIP_REQUIRE(ctx && x && y && tables, "lut_per_channel: NULL argument");
  TPUHIP_REQUIRE(c > 0 && cs >= c && cs % 16 == 0, "lut_per_channel: bad channels %d / stride %d", c, cs);
  if (pixels == 0) return TPUHIP_OK;
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const int64_t total = (int64_t)pixels * (cs / 16);
  launch(ctx, lut_per_channel_kernel, dim3(grid_for(total, kThreads * 2)), dim3(kThreads),
         (const int8_t *)x, (int8_t *)y, (const uint8_t *)tables, total, c, cs);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_prelu_tables(const float *slope, int c, uint32_t rshift_pos, uint32_t multiplier_pos,
                        uint32_t rshift_neg, int8_t *tables) {
  TPUHIP_REQUIRE(slope && tables && c > 0, "prelu_tables: bad argument");
  TPUHIP_REQUIRE(rshift_pos <= 30 && rshift_neg <= 30, "prelu: rshift outside [0,30]");
  // PReluOpKernel::invoke (core/activation.cpp:185-224) for each channel and each of the 256 inputs
  for (int ch = 0; ch < c; ++ch)
    for (int v = -128; v <= 127; ++v) {
      int8_t out;
      if (v > 0) {
        out = host_mult_rshift_sat8((float)v, rshift_pos, multiplier_pos);
      } else {
        volatile float prod = slope[ch] * (float)v;
        volatile float quo = prod / (float)(1 << rshift_neg);
        double s = std::floor((double)quo + 0.5);
        s = s > 127.0 ? 127.0 : s < -128.0 ? -128.0 : s;
        out = (int8_t)(int)s;
      }
      tables[(size_t)ch * 256 + (uint8_t)(int8_t)v] = out;
    }
  return TPUHIP_OK;
}

int tpuhip_leaky_relu_table(uint32_t rshift_pos, uint32_t multiplier_pos, uint32_t rshift_neg,
                            uint32_t multiplier_neg, int8_t *table256) {
  TPUHIP_REQUIRE(table256, "leaky_relu_table: NULL table");
  TPUHIP_REQUIRE(rshift_pos <= 30 && rshift_neg <= 30, "leaky_relu: rshift outside [0,30]");
  // LeakyReluOpKernel::invoke (core/activation.cpp:126-153) for each of the 256 inputs;
  // entry index = two's-complement byte of the input
  for (int v = -128; v <= 127; ++v) {
    int8_t out;
    if (v > 0)
      out = multiplier_pos != 0 ? host_mult_rshift_sat8((float)v, rshift_pos, multiplier_pos)
                                : (int8_t)v;
    else
      out = host_mult_rshift_sat8((float)v, rshift_neg, multiplier_neg);
    table256[(uint8_t)(int8_t)v] = out;
  }
  return TPUHIP_OK;
}

int tpuhip_clip_table(float minv, float maxv, uint32_t rshift, uint32_t multiplier,
                      int8_t *table256) {
  TPUHIP_REQUIRE(table256, "clip_table: NULL table");
  TPUHIP_REQUIRE(rshift <= 30, "clip: rshift outside [0,30]");
  for (int v = -128; v <= 127; ++v) {
    const float c = std::max(minv, std::min((float)v, maxv));
    table256[(uint8_t)(int8_t)v] = host_mult_rshift_sat8(c, rshift, multiplier);
  }
  return TPUHIP_OK;
}

int tpuhip_leaky_relu_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t pixels, int c, int cs,
                         uint32_t rshift_pos, uint32_t multiplier_pos, uint32_t rshift_neg,
                         uint32_t multiplier_neg) {
  int8_t table[256];
  if (int rc = tpuhip_leaky_relu_table(rshift_pos, multiplier_pos, rshift_neg, multiplier_neg,
                                       table))
    return rc;
  return tpuhip_lut_i8(ctx, x, y, table, pixels, c, cs);
}

int tpuhip_relu_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t bytes) {
  TPUHIP_REQUIRE(ctx && x && y, "relu: NULL argument");
  TPUHIP_REQUIRE(bytes % 16 == 0, "relu: byte count %zu not a multiple of 16", bytes);
  if (bytes == 0) return TPUHIP_OK;
  const int64_t n16 = (int64_t)(bytes / 16);
  launch(ctx, relu_kernel, dim3(grid_for(n16, kThreads * 2)), dim3(kThreads), (const v4i *)x, (v4i *)y, n16);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_upsample_nearest_i8(tpuhip_ctx *ctx, const void *x, void *y, int n, int c, int ih,
                               int iw, int scale_h, int scale_w, int x_cs, int y_cs) {
  TPUHIP_REQUIRE(ctx && x && y, "upsample: NULL argument");
  TPUHIP_REQUIRE(n > 0 && c > 0 && ih > 0 && iw > 0 && scale_h > 0 && scale_w > 0,
                 "upsample: non-positive dimension");
  TPUHIP_REQUIRE(x_cs % 16 == 0 && y_cs % 16 == 0 && x_cs >= c && y_cs >= c,
                 "upsample: bad channel strides %d / %d for %d channels", x_cs, y_cs, c);
  const int c16 = (c + 15) / 16;
  const int64_t total = (int64_t)n * ih * scale_h * iw * scale_w * c16;
  launch(ctx, upsample_kernel, dim3(grid_for(total, kThreads * 2)), dim3(kThreads), (const int8_t *)x, (int8_t *)y, n, ih, iw, scale_h, scale_w, c16,
                     x_cs, y_cs);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_concat_i8(tpuhip_ctx *ctx, const void *const *xs, int nin, const int *in_dims,
                     const int *in_cs, int axis, const uint32_t *rshift,
                     const uint32_t *multiplier, int do_relu, void *y, int y_cs) {
  TPUHIP_REQUIRE(ctx && xs && in_dims && in_cs && y, "concat: NULL argument");
  TPUHIP_REQUIRE(nin >= 1, "concat: no inputs");
  TPUHIP_REQUIRE(axis >= 0 && axis <= 3, "concat: axis %d outside 0..3", axis);
  const bool need_quant = rshift != nullptr && multiplier != nullptr;
  int out_dims[4] = {in_dims[0], in_dims[1], in_dims[2], in_dims[3]};
  out_dims[axis] = 0;
  for (int i = 0; i < nin; ++i) {
    TPUHIP_REQUIRE(xs[i], "concat: input %d is NULL", i);
    for (int k = 0; k < 4; ++k) {
      TPUHIP_REQUIRE(in_dims[4 * i + k] > 0, "concat: input %d has a non-positive dimension", i);
      if (k != axis)
        TPUHIP_REQUIRE(in_dims[4 * i + k] == in_dims[k], "concat: input %d differs on axis %d", i, k);
    }
    TPUHIP_REQUIRE(in_cs[i] >= in_dims[4 * i + 1] && in_cs[i] % 16 == 0,
                   "concat: bad channel stride of input %d", i);
    if (need_quant) TPUHIP_REQUIRE(rshift[i] <= 30, "concat: rshift[%d] outside [0,30]", i);
    out_dims[axis] += in_dims[4 * i + axis];
  }
  const int N = out_dims[0], Cc = out_dims[1], H = out_dims[2], W = out_dims[3];
  TPUHIP_REQUIRE(y_cs >= Cc && y_cs % 16 == 0, "concat: bad output channel stride %d", y_cs);

  // A concat that changes no byte (no rescaling that is not the identity; a ReLU would change negative
  // bytes) of two to four inputs is one launch for all of them: along the channels when every input
  // has whole 16-channel groups; along n, h or w when all tensors have the channel stride of their channel count (a chunk
  // is then a run of whole pixels, pad channels included, which are zero in every input).
  bool plain = nin >= 2 && nin <= 4 && !do_relu;
  for (int i = 0; i < nin && plain; ++i) {
    plain = axis == 1 ? in_dims[4 * i + 1] % 16 == 0 : (in_cs[i] == y_cs && y_cs == round_up(Cc, 16));
    if (need_quant && !(multiplier[i] == 1 && rshift[i] == 0)) plain = false;
  }
  if (plain) {
    ConcatArgs a{};
    a.y = (int8_t *)y;
    a.n = nin;
    // bytes of one step along the axis, and of everything inside one outer index of the output
    const int64_t unit = axis == 1 ? 1 : axis == 3 ? y_cs : axis == 2 ? (int64_t)W * y_cs : (int64_t)H * W * y_cs;
    a.outer = axis == 1 ? (int64_t)N * H * W : axis == 3 ? (int64_t)N * H : axis == 2 ? N : 1;
    a.y_stride = axis == 1 ? y_cs : unit * out_dims[axis];
    for (int i = 0; i < nin; ++i) {
      a.x[i] = (const int8_t *)xs[i];
      a.stride[i] = axis == 1 ? in_cs[i] : unit * in_dims[4 * i + axis];
      a.start[i + 1] = a.start[i] + unit * in_dims[4 * i + axis] / 16;
    }
    // the chunks of an outer index fill the output's: Cc channels of a pixel, or all of its rows / pixels
    TPUHIP_REQUIRE(a.start[nin] * 16 == unit * out_dims[axis] && a.start[nin] * 16 <= a.y_stride,
                   "concat: chunks of %lld groups do not fill axis %d", (long long)a.start[nin], axis);
    TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
    // along the channels the output's stride may be wider than its channels: the pad groups are written as zero
    a.groups = axis == 1 ? y_cs / 16 : a.start[nin];
    launch(ctx, concat_chunks_kernel, dim3(grid_for(a.outer * a.groups, kThreads * 4)), dim3(kThreads), a);
    TPUHIP_CHECK_HIP(hipGetLastError());
    return TPUHIP_OK;
  }

  // Each input goes through a 256-entry table: requant (unless m == 1, r == 0) then ReLU
  // -- both pure functions of the int8 input (core/concat.cpp:66-88).
  int offset = 0;  // running offset along the concat axis
  for (int i = 0; i < nin; ++i) {
    const int *dm = in_dims + 4 * i;
    int8_t table[256];
    bool identity = true;
    for (int v = -128; v <= 127; ++v) {
      int8_t o = (int8_t)v;
      if (need_quant && !(multiplier[i] == 1 && rshift[i] == 0))
        o = host_mult_rshift_sat8((float)v, rshift[i], multiplier[i]);
      if (do_relu && o < 0) o = 0;
      if (o != (int8_t)v) identity = false;
      table[(uint8_t)(int8_t)v] = o;
    }
    const int8_t *tab = identity ? nullptr : table;
    const int8_t *src = (const int8_t *)xs[i];
    int8_t *dst = (int8_t *)y;
    int rc = TPUHIP_OK;
    if (axis == 1) {
      rc = launch_lut(ctx, src, dst, tab, (int64_t)N * H * W, dm[1], in_cs[i], y_cs, offset);
    } else if (axis == 0) {
      rc = launch_lut(ctx, src, dst + (int64_t)offset * H * W * y_cs, tab, (int64_t)dm[0] * H * W,
                      Cc, in_cs[i], y_cs, 0);
    } else if (axis == 2) {
      for (int b = 0; b < N && !rc; ++b)
        rc = launch_lut(ctx, src + (int64_t)b * dm[2] * W * in_cs[i],
                        dst + ((int64_t)b * H + offset) * W * y_cs, tab, (int64_t)dm[2] * W, Cc,
                        in_cs[i], y_cs, 0);
    } else {
      for (int b = 0; b < N * H && !rc; ++b)
        rc = launch_lut(ctx, src + (int64_t)b * dm[3] * in_cs[i],
                        dst + ((int64_t)b * W + offset) * y_cs, tab, dm[3], Cc, in_cs[i], y_cs, 0);
    }
    if (rc) return rc;
    offset += dm[axis];
  }
  // channel concat that ends off a 16 boundary: clear the pad channels
  if (axis == 1 && Cc % 16 != 0) {
    const int c1 = std::min(round_up(Cc, 16), y_cs);
    const int64_t total = (int64_t)N * H * W * (c1 - Cc);
    launch(ctx, zero_channels_kernel, dim3(grid_for(total)), dim3(kThreads), (int8_t *)y, (int64_t)N * H * W, y_cs, Cc, c1);
    TPUHIP_CHECK_HIP(hipGetLastError());
  }
  return TPUHIP_OK;
}

}  // extern "C"

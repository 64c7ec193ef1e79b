// Pure data movement on int8 channels-last tensors: Pad, Crop, Permute, Reorg, Tile,
// Reverse, ShuffleChannel, DepthToSpace, SwapChannel, Dilate, ReflectionPad (core/pad.cpp, crop.cpp, permute.cpp,
// reorg.cpp, tile.cpp, reverse.cpp, shuffle_channel.cpp, depthtospace.cpp, swap_channel.cpp,
// dilate.cpp, reflectionpad.cpp).  Each is an index map from
// the logical (n, c, h, w) of an output element to that of its source; one kernel
// evaluates the map per element and moves the byte.  A lane produces four consecutive
// output channels of a pixel (one dword store); pad channels are written as zero.
#include "common.hpp"

#include <cstring>

using namespace tpuhip;

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
constexpr int kThreads = 256;

struct MoveArgs {
  const int8_t *x;
  int8_t *y;
  int kind;
  int in, ic, ih, iw, ics;
  int on, oc, oh, ow, ocs;
  int p[12];
  int fill;        // the byte of an element without a source (0 except for Dilate)
  int64_t total;   // output pixels * (ocs / 4)
};

// source of output element o = (n, c, h, w); false: the element has none and takes a.fill
__device__ __forceinline__ bool source_of(const MoveArgs &a, const int (&o)[4], int (&s)[4]) {
  switch (a.kind) {
    case TPUHIP_MOVE_PAD_CONST: {
      // p[0..3] where the first kept input element lands, p[4..7] its index, p[8..11] end of
      // the kept input range
      bool inside = true;
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        s[d] = o[d] - a.p[d] + a.p[4 + d];
        inside = inside && s[d] >= a.p[4 + d] && s[d] < a.p[8 + d];
      }
      return inside;
    }
    case TPUHIP_MOVE_PAD_EDGE:
      s[0] = o[0];
      s[1] = o[1];
      s[2] = min(max(o[2] - a.p[2], 0), a.ih - 1);
      s[3] = min(max(o[3] - a.p[3], 0), a.iw - 1);
      return true;
    case TPUHIP_MOVE_CROP:
#pragma unroll
      for (int d = 0; d < 4; ++d) s[d] = o[d] * a.p[4 + d] + a.p[d];
      return true;
    case TPUHIP_MOVE_PERMUTE:
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        // output dimension d is input dimension p[d]
#pragma unroll
        for (int k = 0; k < 4; ++k)
          if (a.p[d] == k) s[k] = o[d];
      }
      return true;
    case TPUHIP_MOVE_REORG: {
      const int st = a.p[0], off = o[1] / a.ic;
      s[0] = o[0];
      s[1] = o[1] - off * a.ic;
      s[2] = o[2] * st + off / st;
      s[3] = o[3] * st + off % st;
      return true;
    }
    case TPUHIP_MOVE_TILE: {
      const int dims[4] = {a.in, a.ic, a.ih, a.iw};
#pragma unroll
      for (int d = 0; d < 4; ++d) s[d] = a.p[0] == d ? o[d] % dims[d] : o[d];
      return true;
    }
    case TPUHIP_MOVE_REVERSE: {
      const int dims[4] = {a.in, a.ic, a.ih, a.iw};
#pragma unroll
      for (int d = 0; d < 4; ++d) s[d] = a.p[0] == d ? dims[d] - 1 - o[d] : o[d];
      return true;
    }
    case TPUHIP_MOVE_SHUFFLE_CHANNEL: {
      const int group = a.p[0], col = a.ic / group;
      s[0] = o[0];
      s[1] = (o[1] % group) * col + o[1] / group;
      s[2] = o[2];
      s[3] = o[3];
      return true;
    }
    case TPUHIP_MOVE_SWAP_CHANNEL:
      s[0] = o[0];
      s[1] = o[1];
#pragma unroll
      for (int k = 0; k < 8; ++k)
        if (o[1] == k) s[1] = a.p[k];
      s[2] = o[2];
      s[3] = o[3];
      return true;
    case TPUHIP_MOVE_DILATE: {
      // p[0] = ins_w + 1, p[1] = ins_h + 1: input elements sit on that grid
      const int qh = o[2] / a.p[1], qw = o[3] / a.p[0];
      s[0] = o[0];
      s[1] = o[1];
      s[2] = qh;
      s[3] = qw;
      return qh * a.p[1] == o[2] && qw * a.p[0] == o[3];
    }
    case TPUHIP_MOVE_REFLECTION_PAD: {
      // p[0] = columns added on the left; mirrored about the first / last column
      const int j = o[3] - a.p[0];
      s[0] = o[0];
      s[1] = o[1];
      s[2] = o[2];
      s[3] = j < 0 ? -j : j >= a.iw ? 2 * (a.iw - 1) - j : j;
      return true;
    }
    default: {   // TPUHIP_MOVE_DEPTH_TO_SPACE: p[0] = upscale factor, p[1] = DCR mode
      const int r = a.p[0];
      const int dh = o[2] % r, dw = o[3] % r;
      s[0] = o[0];
      s[1] = a.p[1] ? (dh * r + dw) * a.oc + o[1] : o[1] * r * r + dh * r + dw;
      s[2] = o[2] / r;
      s[3] = o[3] / r;
      return true;
    }
  }
}

__global__ __launch_bounds__(kThreads) void move_kernel(MoveArgs a) {
  const int c4 = a.ocs >> 2;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cq = (int)(i % c4);
    const int pix = (int)(i / c4);
    const int w = pix % a.ow;
    const int h = (pix / a.ow) % a.oh;
    const int n = pix / (a.ow * a.oh);
    uint32_t word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int c = cq * 4 + b;
      if (c >= a.oc) continue;
      const int o[4] = {n, c, h, w};
      int s[4] = {0, 0, 0, 0};
      const int8_t v = source_of(a, o, s)
                           ? a.x[((int64_t)(s[0] * a.ih + s[2]) * a.iw + s[3]) * a.ics + s[1]]
                           : (int8_t)a.fill;
      word |= (uint32_t)(uint8_t)v << (8 * b);
    }
    *reinterpret_cast<uint32_t *>(a.y + (int64_t)pix * a.ocs + cq * 4) = word;
  }
}

// QuantOp at the graph edges (core/quant.cpp).  The float side is NCHW like the reference's
// tensors, the int8 side channels-last: the layout change rides along.
__device__ __forceinline__ float bf16_rne(float v) {   // QuantizationArithmetic.cpp:893-905
  uint32_t u = __float_as_uint(v);
  u += 0x7fffu + ((u >> 16) & 1u);
  uint32_t h = u >> 16;
  if ((h & 0x7f80u) == 0x7f80u) h = 0x7f7fu;
  return __uint_as_float(h << 16);
}

__global__ __launch_bounds__(kThreads) void quant_f32_to_i8_kernel(const float *x, int8_t *y, int n,
                                                                   int c, int h, int w, int cs,
                                                                   float scale) {
  const int64_t total = (int64_t)n * h * w * cs;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int ch = (int)(i % cs);
    const int64_t pix = i / cs;
    int8_t out = 0;
    if (ch < c) {
      const int iw = (int)(pix % w), ih = (int)((pix / w) % h), in = (int)(pix / ((int64_t)w * h));
      const float v = x[(((int64_t)in * c + ch) * h + ih) * w + iw];
      const float r = roundf(__fmul_rn(v, scale));   // std::round: half away from zero
      out = (int8_t)(r > 127.0f ? 127 : r < -128.0f ? -128 : (int)r);
    }
    y[i] = out;
  }
}

__global__ __launch_bounds__(kThreads) void dequant_i8_to_f32_kernel(const int8_t *x, float *y,
                                                                     int n, int c, int h, int w,
                                                                     int cs, float scale_bf16) {
  const int64_t total = (int64_t)n * c * h * w;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int iw = (int)(i % w), ih = (int)((i / w) % h);
    const int ch = (int)((i / ((int64_t)w * h)) % c), in = (int)(i / ((int64_t)w * h * c));
    const float v = (float)x[(((int64_t)in * h + ih) * w + iw) * cs + ch];   // exact in bf16
    y[i] = bf16_rne(__fmul_rn(v, scale_bf16));
  }
}

}  // namespace

extern "C" int tpuhip_quant_f32_to_i8(tpuhip_ctx *ctx, const void *x_nchw_f32, void *y, int n, int c,
                                      int h, int w, int cs, float scale) {
  TPUHIP_REQUIRE(ctx && x_nchw_f32 && y, "quant: NULL argument");
  TPUHIP_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && cs >= c && cs % 16 == 0, "quant: bad shape");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const int64_t total = (int64_t)n * h * w * cs;
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(total, kThreads), (int64_t)ctx->num_cu * 32));
  launch(ctx, quant_f32_to_i8_kernel, dim3(blocks), dim3(kThreads), (const float *)x_nchw_f32,
         (int8_t *)y, n, c, h, w, cs, scale);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

extern "C" int tpuhip_dequant_i8_to_f32(tpuhip_ctx *ctx, const void *x, void *y_nchw_f32, int n, int c,
                                        int h, int w, int cs, float scale) {
  TPUHIP_REQUIRE(ctx && x && y_nchw_f32, "dequant: NULL argument");
  TPUHIP_REQUIRE(n > 0 && c > 0 && h > 0 && w > 0 && cs >= c && cs % 16 == 0, "dequant: bad shape");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  // scale = BF16(scale) on the host (quant.cpp:110), same rounding as the device function
  uint32_t u;
  memcpy(&u, &scale, 4);
  u += 0x7fffu + ((u >> 16) & 1u);
  uint32_t hbits = u >> 16;
  if ((hbits & 0x7f80u) == 0x7f80u) hbits = 0x7f7fu;
  hbits <<= 16;
  float sb;
  memcpy(&sb, &hbits, 4);
  const int64_t total = (int64_t)n * c * h * w;
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(total, kThreads), (int64_t)ctx->num_cu * 32));
  launch(ctx, dequant_i8_to_f32_kernel, dim3(blocks), dim3(kThreads), (const int8_t *)x,
         (float *)y_nchw_f32, n, c, h, w, cs, sb);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

namespace {

// Reduce over consecutive logical (NCHW) axes: kind 0 mean / 1 sum / 2 max / 3 min
// (core/reduce.cpp:54-117, INT8).  A lane produces four consecutive channels of an output
// pixel; each walks its `axis` sources through the logical index map.
struct ReduceArgs {
  const int8_t *x;
  int8_t *y;
  int kind, requant;
  int ic, ih, iw, ics;
  int oc, oh, ow, ocs;
  int axis, inner;
  float mult, inv_pot;
  int64_t total;   // output pixels * (ocs / 4)
};

__global__ __launch_bounds__(kThreads) void reduce_kernel(ReduceArgs a) {
  const int c4 = a.ocs >> 2;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < a.total;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int cq = (int)(i % c4);
    const int pix = (int)(i / c4);
    const int w = pix % a.ow;
    const int h = (pix / a.ow) % a.oh;
    const int n = pix / (a.ow * a.oh);
    uint32_t word = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int c = cq * 4 + b;
      if (c >= a.oc) continue;
      // logical flat index of the output element, split at the reduced axes
      const int64_t e = (((int64_t)n * a.oc + c) * a.oh + h) * a.ow + w;
      const int64_t o = e / a.inner, in = e - o * a.inner;
      int acc = a.kind == 2 ? -128 : a.kind == 3 ? 127 : 0;
      for (int k = 0; k < a.axis; ++k) {
        const int64_t l = (o * a.axis + k) * a.inner + in;
        const int sw = (int)(l % a.iw);
        const int64_t t1 = l / a.iw;
        const int sh = (int)(t1 % a.ih);
        const int64_t t2 = t1 / a.ih;
        const int sc = (int)(t2 % a.ic);
        const int64_t sn = t2 / a.ic;
        const int v = a.x[((sn * a.ih + sh) * a.iw + sw) * a.ics + sc];
        acc = a.kind <= 1 ? acc + v : a.kind == 2 ? max(acc, v) : min(acc, v);
      }
      int r = acc;
      if (a.requant) {
        // the float overload of applyMultiplierAndRShiftAndSaturateInt8 without qdm
        const float prod = __fmul_rn((float)acc, a.mult);
        r = saturate_int8_f(__fmul_rn(prod, a.inv_pot));   // power-of-two scaling: exact
      }
      word |= (uint32_t)(uint8_t)(int8_t)r << (8 * b);
    }
    *reinterpret_cast<uint32_t *>(a.y + (int64_t)pix * a.ocs + cq * 4) = word;
  }
}

}  // namespace

extern "C" int tpuhip_reduce_i8(tpuhip_ctx *ctx, int kind, const void *x, void *y, const int *in_nchw,
                                int x_cs, const int *out_nchw, int y_cs, int first_axis, int last_axis,
                                int rshift, uint32_t multiplier) {
  TPUHIP_REQUIRE(ctx && x && y && in_nchw && out_nchw, "reduce: NULL argument");
  TPUHIP_REQUIRE(kind >= 0 && kind <= 3, "reduce: unknown kind %d", kind);
  TPUHIP_REQUIRE(first_axis >= 0 && first_axis <= last_axis && last_axis < 4, "reduce: axes %d..%d", first_axis,
                 last_axis);
  int64_t outer = 1, axis = 1, inner = 1, out_count = 1;
  for (int k = 0; k < 4; ++k) {
    TPUHIP_REQUIRE(in_nchw[k] > 0 && out_nchw[k] > 0, "reduce: non-positive dimension");
    (k < first_axis ? outer : k <= last_axis ? axis : inner) *= in_nchw[k];
    out_count *= out_nchw[k];
  }
  TPUHIP_REQUIRE(out_count == outer * inner, "reduce: the result holds %lld elements, expected %lld",
                 (long long)out_count, (long long)(outer * inner));
  TPUHIP_REQUIRE(x_cs >= in_nchw[1] && x_cs % 16 == 0 && y_cs >= out_nchw[1] && y_cs % 16 == 0,
                 "reduce: channel strides must be multiples of 16 covering the channels");
  TPUHIP_REQUIRE(outer * axis * inner < (1ll << 31) && axis * 128 < (1ll << 24),
                 "reduce: tensor too large (the reference's float sum must stay exact)");
  TPUHIP_REQUIRE(rshift >= 0 && rshift <= 30, "reduce: rshift %d outside [0,30]", rshift);
  const bool requant = rshift != 0 || multiplier != 1;
  TPUHIP_REQUIRE(requant || kind >= 2 || axis == 1,
                 "reduce: a sum with rshift 0 and multiplier 1 has no int8 value (the reference leaves "
                 "the raw sum in its float tensor)");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  ReduceArgs a{};
  a.x = (const int8_t *)x;
  a.y = (int8_t *)y;
  a.kind = kind;
  a.requant = requant ? 1 : 0;
  a.ic = in_nchw[1]; a.ih = in_nchw[2]; a.iw = in_nchw[3]; a.ics = x_cs;
  a.oc = out_nchw[1]; a.oh = out_nchw[2]; a.ow = out_nchw[3]; a.ocs = y_cs;
  a.axis = (int)axis;
  a.inner = (int)inner;
  a.mult = (float)multiplier;
  a.inv_pot = 1.0f / (float)(1u << rshift);
  a.total = (int64_t)out_nchw[0] * out_nchw[2] * out_nchw[3] * (y_cs / 4);
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(a.total, kThreads), (int64_t)ctx->num_cu * 32));
  launch(ctx, reduce_kernel, dim3(blocks), dim3(kThreads), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

namespace {

// ---------------------------------------------------------------------------
// Permute without the per-byte index map.  S[k]: byte stride of input dimension k in the input,
// T[k]: byte stride, in the output, of the output dimension that input dimension k becomes.
// ---------------------------------------------------------------------------
struct PermArgs {
  const int8_t *x;
  int8_t *y;
  int dim[4];        // input dimensions (n, c, h, w)
  int64_t S[4], T[4];
  int ocs;           // channel stride of the output
  int ics;           // channel stride of the input
  int j, a, b;       // j: the input dimension that becomes the output's channels; a, b: the other two besides c
};

// channels stay channels (j == 1): a pixel's channel row moves as 16-byte chunks.  The two channel
// strides may differ (a padded stride on either side): groups of the output row beyond the input's
// stride are written as zero, never read from the next pixel.
__global__ __launch_bounds__(kThreads) void permute_rows_kernel(PermArgs q, int64_t total) {
  const int c16 = q.ocs >> 4;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(i % c16);
    int64_t pix = i / c16;                       // input pixel (n, h, w) in input order
    const int w = (int)(pix % q.dim[3]);
    pix /= q.dim[3];
    const int h = (int)(pix % q.dim[2]);
    const int n = (int)(pix / q.dim[2]);
    v4i v = {0, 0, 0, 0};
    if (cg * 16 < q.ics) v = *reinterpret_cast<const v4i *>(q.x + n * q.S[0] + h * q.S[2] + w * q.S[3] + cg * 16);
    *reinterpret_cast<v4i *>(q.y + n * q.T[0] + h * q.T[2] + w * q.T[3] + cg * 16) = v;
  }
}

// the channels change places with dimension j: 64 x 64 byte tiles through LDS, dword loads along
// the input's channels, dword stores along the output's (pad channels of the output written as
// zero: tile rows past the end of dimension j are zero)
__global__ __launch_bounds__(kThreads) void permute_tile_kernel(PermArgs q) {
  __shared__ __attribute__((aligned(4))) int8_t tile[64][68];
  const int c0 = blockIdx.y * 64, j0 = blockIdx.x * 64;
  const int ia = (int)(blockIdx.z / q.dim[q.b]), ib = (int)(blockIdx.z % q.dim[q.b]);
  const int8_t *src = q.x + ia * q.S[q.a] + ib * q.S[q.b];
  int8_t *dst = q.y + ia * q.T[q.a] + ib * q.T[q.b];
  const int tq = threadIdx.x & 15, tr = threadIdx.x >> 4;   // 16 dwords per row, 16 rows per pass
#pragma unroll
  for (int r = tr; r < 64; r += 16) {
    const int jj = j0 + r, cc = c0 + tq * 4;
    uint32_t v = 0;
    // the input's pad channels are zero and its channel stride is a multiple of 16, so a dword
    // that starts inside the row may be read whole
    if (jj < q.dim[q.j] && cc < q.dim[1]) v = *reinterpret_cast<const uint32_t *>(src + jj * q.S[q.j] + cc);
    *reinterpret_cast<uint32_t *>(&tile[r][tq * 4]) = v;
  }
  __syncthreads();
#pragma unroll
  for (int r = tr; r < 64; r += 16) {
    const int cc = c0 + r, jj = j0 + tq * 4;
    if (cc < q.dim[1] && jj < q.ocs) {
      const uint32_t v = (uint32_t)(uint8_t)tile[tq * 4][r] | ((uint32_t)(uint8_t)tile[tq * 4 + 1][r] << 8) |
                         ((uint32_t)(uint8_t)tile[tq * 4 + 2][r] << 16) | ((uint32_t)(uint8_t)tile[tq * 4 + 3][r] << 24);
      *reinterpret_cast<uint32_t *>(dst + cc * q.T[1] + jj) = v;
    }
  }
}

// permute of dense row-major bytes over the full rank (at most 6): a lane owns an output element
struct FlatPermArgs {
  const int8_t *x;
  int8_t *y;
  int rank;
  int oshape[6];
  int64_t istr[6];   // input stride of the input dimension that output dimension d is
  int64_t total;
};
__global__ __launch_bounds__(kThreads) void permute_flat_kernel(FlatPermArgs q) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < q.total; i += (int64_t)gridDim.x * blockDim.x) {
    int64_t r = i, off = 0;
    for (int d = q.rank - 1; d >= 0; --d) {
      const int64_t c = r % q.oshape[d];
      r /= q.oshape[d];
      off += c * q.istr[d];
    }
    q.y[i] = q.x[off];
  }
}

int run_permute(tpuhip_ctx *ctx, const tpuhip_move_desc *d, const void *x, void *y) {
  PermArgs q{};
  q.x = (const int8_t *)x;
  q.y = (int8_t *)y;
  q.dim[0] = d->in; q.dim[1] = d->ic; q.dim[2] = d->ih; q.dim[3] = d->iw;
  q.S[0] = (int64_t)d->ih * d->iw * d->x_cs; q.S[1] = 1; q.S[2] = (int64_t)d->iw * d->x_cs; q.S[3] = d->x_cs;
  const int64_t tout[4] = {(int64_t)d->oh * d->ow * d->y_cs, 1, (int64_t)d->ow * d->y_cs, d->y_cs};
  for (int k = 0; k < 4; ++k) q.T[d->p[k]] = tout[k];   // output dimension k is input dimension p[k]
  q.ocs = d->y_cs;
  q.ics = d->x_cs;
  q.j = d->p[1];
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  if (q.j == 1) {
    const int64_t total = (int64_t)d->in * d->ih * d->iw * (d->y_cs / 16);
    const unsigned blocks = (unsigned)std::max<int64_t>(
        1, std::min<int64_t>(ceil_div64(total, kThreads), (int64_t)ctx->num_cu * 32));
    launch(ctx, permute_rows_kernel, dim3(blocks), dim3(kThreads), q, total);
  } else {
    int rest[2], nr = 0;
    for (int k = 0; k < 4; ++k)
      if (k != 1 && k != q.j) rest[nr++] = k;
    q.a = rest[0];
    q.b = rest[1];
    const int64_t batch = (int64_t)q.dim[q.a] * q.dim[q.b];
    TPUHIP_REQUIRE(batch <= 65535, "permute: more than 65535 planes (%lld)", (long long)batch);
    const dim3 grid((unsigned)((d->y_cs + 63) / 64), (unsigned)((d->ic + 63) / 64), (unsigned)batch);
    launch(ctx, permute_tile_kernel, grid, dim3(kThreads), q);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // namespace

extern "C" int tpuhip_move_i8(tpuhip_ctx *ctx, const tpuhip_move_desc *d, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && d && x && y, "move: NULL argument");
  TPUHIP_REQUIRE(d->kind >= TPUHIP_MOVE_PAD_CONST && d->kind <= TPUHIP_MOVE_REFLECTION_PAD,
                 "move: unknown kind %d", d->kind);
  TPUHIP_REQUIRE(d->in > 0 && d->ic > 0 && d->ih > 0 && d->iw > 0 && d->on > 0 && d->oc > 0 &&
                     d->oh > 0 && d->ow > 0,
                 "move: non-positive dimension");
  TPUHIP_REQUIRE(d->x_cs >= d->ic && d->x_cs % 16 == 0 && d->y_cs >= d->oc && d->y_cs % 16 == 0,
                 "move: channel strides must be multiples of 16 covering the channels");
  TPUHIP_REQUIRE((int64_t)d->in * d->ih * d->iw * d->x_cs < (1ll << 31) &&
                     (int64_t)d->on * d->oh * d->ow < (1ll << 31),
                 "move: tensor too large");
  const int is[4] = {d->in, d->ic, d->ih, d->iw}, os[4] = {d->on, d->oc, d->oh, d->ow};
  const int *p = d->p;
  MoveArgs a{};
  // every kind: check that the map stays inside the input for every output element
  switch (d->kind) {
    case TPUHIP_MOVE_PAD_CONST:
      // p[0..3] pads at the beginning, p[4..7] at the end (negative: cut), as the op's attribute
      for (int k = 0; k < 4; ++k) {
        TPUHIP_REQUIRE(os[k] == is[k] + p[k] + p[4 + k], "pad: output dimension %d is %d, expected %d",
                       k, os[k], is[k] + p[k] + p[4 + k]);
        a.p[k] = p[k] < 0 ? 0 : p[k];
        a.p[4 + k] = p[k] < 0 ? -p[k] : 0;
        a.p[8 + k] = p[4 + k] < 0 ? is[k] + p[4 + k] : is[k];
        TPUHIP_REQUIRE(a.p[4 + k] <= a.p[8 + k], "pad: dimension %d is cut away entirely", k);
      }
      break;
    case TPUHIP_MOVE_PAD_EDGE:
      TPUHIP_REQUIRE(p[0] == 0 && p[1] == 0 && p[4] == 0 && p[5] == 0, "pad: edge mode pads h and w only");
      TPUHIP_REQUIRE(p[2] >= 0 && p[3] >= 0 && p[6] >= 0 && p[7] >= 0, "pad: edge mode needs pads >= 0");
      for (int k = 0; k < 4; ++k) {
        TPUHIP_REQUIRE(os[k] == is[k] + p[k] + p[4 + k], "pad: output dimension %d is %d, expected %d",
                       k, os[k], is[k] + p[k] + p[4 + k]);
        a.p[k] = p[k];
      }
      break;
    case TPUHIP_MOVE_CROP:
      // p[0..3] offsets, p[4..7] steps
      for (int k = 0; k < 4; ++k) {
        TPUHIP_REQUIRE(p[k] >= 0 && p[4 + k] >= 1 && (int64_t)(os[k] - 1) * p[4 + k] + p[k] < is[k],
                       "crop: dimension %d reads past the input", k);
        a.p[k] = p[k];
        a.p[4 + k] = p[4 + k];
      }
      break;
    case TPUHIP_MOVE_PERMUTE: {
      int seen = 0;
      for (int k = 0; k < 4; ++k) {
        TPUHIP_REQUIRE(p[k] >= 0 && p[k] < 4, "permute: order[%d] = %d", k, p[k]);
        seen |= 1 << p[k];
        TPUHIP_REQUIRE(os[k] == is[p[k]], "permute: output dimension %d is %d, expected %d", k, os[k],
                       is[p[k]]);
        a.p[k] = p[k];
      }
      TPUHIP_REQUIRE(seen == 15, "permute: order is not a permutation");
      // tiled kernels; the per-byte map below serves the other kinds (and permutes with more
      // planes than a launch grid holds)
      if (p[1] == 1 || (int64_t)is[0] * is[2] * is[3] / is[p[1]] <= 65535) return run_permute(ctx, d, x, y);
      break;
    }
    case TPUHIP_MOVE_REORG:
      TPUHIP_REQUIRE(p[0] >= 1 && is[2] % p[0] == 0 && is[3] % p[0] == 0, "reorg: bad stride %d", p[0]);
      TPUHIP_REQUIRE(os[0] == is[0] && os[1] == is[1] * p[0] * p[0] && os[2] == is[2] / p[0] &&
                         os[3] == is[3] / p[0],
                     "reorg: output shape does not match");
      a.p[0] = p[0];
      break;
    case TPUHIP_MOVE_TILE:
      TPUHIP_REQUIRE(p[0] >= 0 && p[0] < 4 && p[1] >= 1, "tile: bad axis %d / tiles %d", p[0], p[1]);
      for (int k = 0; k < 4; ++k)
        TPUHIP_REQUIRE(os[k] == (k == p[0] ? is[k] * p[1] : is[k]), "tile: output dimension %d is %d", k,
                       os[k]);
      a.p[0] = p[0];
      break;
    case TPUHIP_MOVE_REVERSE:
      TPUHIP_REQUIRE(p[0] >= 0 && p[0] < 4, "reverse: bad axis %d", p[0]);
      for (int k = 0; k < 4; ++k) TPUHIP_REQUIRE(os[k] == is[k], "reverse: shapes differ");
      a.p[0] = p[0];
      break;
    case TPUHIP_MOVE_SHUFFLE_CHANNEL:
      TPUHIP_REQUIRE(p[0] >= 1 && is[1] % p[0] == 0, "shuffle_channel: wrong group size, c=%d, group=%d",
                     is[1], p[0]);
      for (int k = 0; k < 4; ++k) TPUHIP_REQUIRE(os[k] == is[k], "shuffle_channel: shapes differ");
      a.p[0] = p[0];
      break;
    case TPUHIP_MOVE_SWAP_CHANNEL:
      TPUHIP_REQUIRE(is[1] <= 8, "swap_channel: at most 8 channels (%d)", is[1]);
      for (int k = 0; k < 4; ++k) TPUHIP_REQUIRE(os[k] == is[k], "swap_channel: shapes differ");
      for (int k = 0; k < is[1]; ++k) {
        TPUHIP_REQUIRE(p[k] >= 0 && p[k] < is[1], "swap_channel: channel_order[%d] = %d", k, p[k]);
        a.p[k] = p[k];
      }
      break;
    case TPUHIP_MOVE_DILATE:
      // p[0] = ins_w, p[1] = ins_h, p[2] = fill_constant
      TPUHIP_REQUIRE(p[0] >= 0 && p[1] >= 0, "dilate: negative ins (%d, %d)", p[0], p[1]);
      TPUHIP_REQUIRE(p[2] >= -128 && p[2] <= 127, "dilate: fill_constant %d is no int8 value", p[2]);
      TPUHIP_REQUIRE(os[0] == is[0] && os[1] == is[1] &&
                         (int64_t)os[2] == (int64_t)(is[2] - 1) * (p[1] + 1) + 1 &&
                         (int64_t)os[3] == (int64_t)(is[3] - 1) * (p[0] + 1) + 1,
                     "dilate: output shape does not match");
      a.p[0] = p[0] + 1;
      a.p[1] = p[1] + 1;
      a.fill = p[2];
      break;
    case TPUHIP_MOVE_REFLECTION_PAD:
      // p[0] / p[1] columns added on the left / right; a mirror image needs a column to mirror
      TPUHIP_REQUIRE(p[0] >= 0 && p[1] >= 0 && p[0] < is[3] && p[1] < is[3],
                     "reflection_pad: pads (%d, %d) must be in [0, w = %d)", p[0], p[1], is[3]);
      TPUHIP_REQUIRE(os[0] == is[0] && os[1] == is[1] && os[2] == is[2] && os[3] == is[3] + p[0] + p[1],
                     "reflection_pad: output shape does not match");
      a.p[0] = p[0];
      break;
    default:
      TPUHIP_REQUIRE(p[0] >= 1 && is[1] % (p[0] * p[0]) == 0, "depth_to_space: bad upscale factor %d", p[0]);
      TPUHIP_REQUIRE(os[0] == is[0] && os[1] == is[1] / (p[0] * p[0]) && os[2] == is[2] * p[0] &&
                         os[3] == is[3] * p[0],
                     "depth_to_space: output shape does not match");
      a.p[0] = p[0];
      a.p[1] = p[1] ? 1 : 0;
      break;
  }
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  a.x = (const int8_t *)x; a.y = (int8_t *)y;
  a.kind = d->kind;
  a.in = d->in; a.ic = d->ic; a.ih = d->ih; a.iw = d->iw; a.ics = d->x_cs;
  a.on = d->on; a.oc = d->oc; a.oh = d->oh; a.ow = d->ow; a.ocs = d->y_cs;
  a.total = (int64_t)d->on * d->oh * d->ow * (d->y_cs / 4);
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(a.total, kThreads), (int64_t)ctx->num_cu * 32));
  launch(ctx, move_kernel, dim3(blocks), dim3(kThreads), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

extern "C" int tpuhip_permute_flat_i8(tpuhip_ctx *ctx, const void *x, void *y, int rank, const int64_t *in_shape,
                                      const int *order) {
  TPUHIP_REQUIRE(ctx && x && y && in_shape && order, "permute_flat: NULL argument");
  TPUHIP_REQUIRE(rank >= 1 && rank <= 6, "permute_flat: rank %d outside [1,6]", rank);
  FlatPermArgs q{};
  q.x = (const int8_t *)x;
  q.y = (int8_t *)y;
  q.rank = rank;
  int64_t istride[6], total = 1;
  int seen = 0;
  for (int d = rank - 1; d >= 0; --d) {
    TPUHIP_REQUIRE(in_shape[d] >= 1 && in_shape[d] < (1ll << 31), "permute_flat: bad dimension %d", d);
    istride[d] = total;
    total *= in_shape[d];
  }
  TPUHIP_REQUIRE(total < (1ll << 31), "permute_flat: tensor too large");
  for (int d = 0; d < rank; ++d) {
    TPUHIP_REQUIRE(order[d] >= 0 && order[d] < rank, "permute_flat: order[%d] = %d", d, order[d]);
    seen |= 1 << order[d];
    q.oshape[d] = (int)in_shape[order[d]];
    q.istr[d] = istride[order[d]];
  }
  TPUHIP_REQUIRE(seen == (1 << rank) - 1, "permute_flat: order is not a permutation");
  q.total = total;
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const unsigned blocks = (unsigned)std::max<int64_t>(
      1, std::min<int64_t>(ceil_div64(total, kThreads), (int64_t)ctx->num_cu * 32));
  launch(ctx, permute_flat_kernel, dim3(blocks), dim3(kThreads), q);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

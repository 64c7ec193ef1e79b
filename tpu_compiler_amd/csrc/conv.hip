// INT8 Conv2D / FullyConnected for gfx950.
//
//   * dense (g == 1) convolutions and FC: implicit GEMM on the int8 MFMA
//     instruction (v_mfma_i32_32x32x32_i8), weights as the A operand (rows =
//     output channels), im2col'ed channels-last activations as the B operand
//     (columns = output pixels), both staged through LDS in 64-byte K slices;
//   * depthwise (g == ic == oc): channels-last direct kernel, no MFMA;
//   * anything else (grouped, input dilation): one thread per output.
//
// All three share the requantisation epilogue of
// quantizeActivationInt8PerChannelMultiplierAndRShift
// (lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp:849-871).
#include "common.hpp"

#include <vector>

using namespace tpuhip;

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

enum ConvAlgo { ALGO_AUTO = 0, ALGO_DIRECT = 1, ALGO_MFMA = 2, ALGO_DEPTHWISE = 3 };

// Per-output-channel epilogue parameters, one 32-byte record per channel so a
// lane fetches a channel's record with two 16-byte loads.
struct __attribute__((aligned(32))) ChanParams {
  int32_t bias;
  int32_t mult;
  int32_t rshift;
  int32_t mask;   // 2^rshift - 1
  int32_t half;   // mask >> 1
  int32_t pad[3];
};

struct tpuhip_conv_weights {
  tpuhip_conv_desc d;
  int algo = ALGO_DIRECT;
  int tile = 0;          // MFMA tile variant
  int8_t *w = nullptr;   // packed filter
  ChanParams *cp = nullptr;
  int ocp = 0;           // padded output channels (rows of w / entries of cp)
  int kp = 0;            // padded K in bytes (row stride of w) for the MFMA path
  int c16 = 0;           // input 16-channel groups per tap
  int k16 = 0;           // 16-byte K groups in total
};

struct ConvArgs {
  const int8_t *x;
  const int8_t *w;
  const ChanParams *cp;
  int8_t *y;
  int n, ih, iw, x_cs;
  int oh, ow, y_cs;
  int oc, ocw, icg, ocg, g;  // ocw = oc rounded up to 16: channels written per pixel
  int kh, kw, sh, sw, pt, pl, dh, dw, ins_h, ins_w;
  int c16, k16, kp;
  int npix;
  int lo;          // lower clamp bound: 0 with ReLU after saturation, else -128
  int relu_first;  // ReLU on the sum before requantisation (FC)
};

__device__ __forceinline__ int32_t epilogue(int32_t acc, const ChanParams &p, int lo,
                                            int relu_first) {
  int32_t v = (int32_t)((uint32_t)acc + (uint32_t)p.bias);
  if (relu_first) v = max(v, 0);
  return requant_qdm(v, p.mult, p.rshift, p.mask, p.half, lo);
}

// ---------------------------------------------------------------------------
// direct kernel: one thread per (pixel, output channel).  Filter layout
// [oc][kh][kw][icg] dense.  Handles groups, dilation and inserted zeros.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void conv_direct_kernel(ConvArgs a) {
  const int64_t total = (int64_t)a.npix * a.ocw;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int oc = (int)(idx % a.ocw);
    const int pix = (int)(idx / a.ocw);
    int8_t *yp = a.y + (int64_t)pix * a.y_cs + oc;
    if (oc >= a.oc) {
      *yp = 0;
      continue;
    }
    const int ow = pix % a.ow;
    const int oh = (pix / a.ow) % a.oh;
    const int n = pix / (a.ow * a.oh);
    const int gi = oc / a.ocg;
    const int ihd = (a.ih - 1) * (a.ins_h + 1) + 1;
    const int iwd = (a.iw - 1) * (a.ins_w + 1) + 1;
    int32_t acc = 0;
    for (int kh = 0; kh < a.kh; ++kh) {
      const int hp = oh * a.sh - a.pt + kh * a.dh;
      if (hp < 0 || hp >= ihd || (hp % (a.ins_h + 1)) != 0) continue;
      const int ih = hp / (a.ins_h + 1);
      for (int kw = 0; kw < a.kw; ++kw) {
        const int wp = ow * a.sw - a.pl + kw * a.dw;
        if (wp < 0 || wp >= iwd || (wp % (a.ins_w + 1)) != 0) continue;
        const int iw = wp / (a.ins_w + 1);
        const int8_t *xp = a.x + ((int64_t)(n * a.ih + ih) * a.iw + iw) * a.x_cs + gi * a.icg;
        const int8_t *wp_ = a.w + (((int64_t)oc * a.kh + kh) * a.kw + kw) * a.icg;
        for (int c = 0; c < a.icg; ++c) acc += (int32_t)xp[c] * (int32_t)wp_[c];
      }
    }
    *yp = (int8_t)epilogue(acc, a.cp[oc], a.lo, a.relu_first);
  }
}

// ---------------------------------------------------------------------------
// depthwise kernel: one thread per (pixel, 16-channel group).  Filter layout
// [kh][kw][ocw] (channel fastest, zero in the pad channels).
// ---------------------------------------------------------------------------
__device__ __forceinline__ int32_t sbyte(int32_t word, int i) {
  return (int32_t)(int8_t)(word >> (8 * i));
}

__global__ __launch_bounds__(256) void conv_depthwise_kernel(ConvArgs a) {
  const int c16 = a.ocw >> 4;
  const int64_t total = (int64_t)a.npix * c16;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int cg = (int)(idx % c16);
    const int pix = (int)(idx / c16);
    const int ow = pix % a.ow;
    const int oh = (pix / a.ow) % a.oh;
    const int n = pix / (a.ow * a.oh);
    int32_t acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[i] = 0;
    for (int kh = 0; kh < a.kh; ++kh) {
      const int ih = oh * a.sh - a.pt + kh * a.dh;
      if (ih < 0 || ih >= a.ih) continue;
      for (int kw = 0; kw < a.kw; ++kw) {
        const int iw = ow * a.sw - a.pl + kw * a.dw;
        if (iw < 0 || iw >= a.iw) continue;
        const v4i xv = *reinterpret_cast<const v4i *>(
            a.x + ((int64_t)(n * a.ih + ih) * a.iw + iw) * a.x_cs + cg * 16);
        const v4i wv = *reinterpret_cast<const v4i *>(
            a.w + ((int64_t)(kh * a.kw + kw)) * a.ocw + cg * 16);
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
          for (int b = 0; b < 4; ++b) acc[q * 4 + b] += sbyte(xv[q], b) * sbyte(wv[q], b);
      }
    }
    v4i out;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      uint32_t word = 0;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int c = cg * 16 + q * 4 + b;
        int32_t v = 0;
        if (c < a.oc) v = epilogue(acc[q * 4 + b], a.cp[c], a.lo, a.relu_first);
        word |= ((uint32_t)v & 0xffu) << (8 * b);
      }
      out[q] = (int)word;
    }
    *reinterpret_cast<v4i *>(a.y + (int64_t)pix * a.y_cs + cg * 16) = out;
  }
}

// ---------------------------------------------------------------------------
// MFMA implicit-GEMM kernel.
//
//   D[oc][pix] = sum_k W[oc][k] * X[pix][k],   k = (kh*KW + kw)*cs_in + c
//
// Workgroup = 4 waves, tile BM output channels x BN pixels, K consumed 64 bytes
// per step.  LDS rows are 64 bytes (4 chunks of 16); chunk index is XOR-swizzled
// with (row >> 2) & 3 so that both the 16-byte stores of the loader and the
// 16-byte fragment reads of the MFMA loop spread over all banks.
// ---------------------------------------------------------------------------
template <int BM, int BN, int WM, int WN>
__global__ __launch_bounds__(256) void conv_mfma_kernel(ConvArgs a) {
  static_assert(WM * WN == 4, "four waves per workgroup");
  constexpr int TM = BM / WM / 32;  // 32x32 blocks per wave along oc
  constexpr int TN = BN / WN / 32;  // 32x32 blocks per wave along pixels
  static_assert(TM >= 1 && TN >= 1, "tile too small");
  constexpr int NW = BM * 4 / 256;  // 16-byte weight chunks per thread per step
  constexpr int NX = BN * 4 / 256;  // 16-byte activation chunks per thread per step
  static_assert(NX >= 1, "pixel tile too small");

  __shared__ v4i lds[2][(BM + BN) * 4];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int oc0 = blockIdx.y * BM;
  const int pix0 = blockIdx.x * BN;

  // ---- loader state: this thread always fetches K-chunk kc of rows (tid>>2)+64*s
  const int kc = tid & 3;
  const int lrow = tid >> 2;
  int64_t xbase[NX];  // byte offset of image n in x
  int ih0[NX], iw0[NX];
  bool pvalid[NX];
#pragma unroll
  for (int s = 0; s < NX; ++s) {
    const int pix = pix0 + lrow + 64 * s;
    pvalid[s] = pix < a.npix;
    const int p = pvalid[s] ? pix : 0;
    const int ow = p % a.ow;
    const int t = p / a.ow;
    const int oh = t % a.oh;
    const int n = t / a.oh;
    xbase[s] = (int64_t)n * a.ih * a.iw * a.x_cs;
    ih0[s] = oh * a.sh - a.pt;
    iw0[s] = ow * a.sw - a.pl;
  }
  // position of this thread's K group inside the filter window
  int kg = kc;                 // 16-byte group index along K
  int cgrp = kc % a.c16;       // 16-channel group inside the tap
  int tap = kc / a.c16;
  int tkh = tap / a.kw, tkw = tap % a.kw;

  const int8_t *wrow[NW > 0 ? NW : 1];
#pragma unroll
  for (int s = 0; s < NW; ++s)
    wrow[s] = a.w + (int64_t)(oc0 + lrow + 64 * s) * a.kp + kc * 16;
  // BM == 32: only threads with lrow < 32 carry a weight chunk
  const bool wsmall = (BM * 4 < 256);
  const int8_t *wrow_small = a.w + (int64_t)(oc0 + (lrow & (BM - 1))) * a.kp + kc * 16;

  v4i wreg[NW > 0 ? NW : 1], xreg[NX];

  auto load_tile = [&](int step) {
    if (wsmall) {
      if (lrow < BM) wreg[0] = *reinterpret_cast<const v4i *>(wrow_small + (int64_t)step * 64);
    } else {
#pragma unroll
      for (int s = 0; s < NW; ++s)
        wreg[s] = *reinterpret_cast<const v4i *>(wrow[s] + (int64_t)step * 64);
    }
    const bool kvalid = kg < a.k16;
    const int dh_off = tkh * a.dh, dw_off = tkw * a.dw;
#pragma unroll
    for (int s = 0; s < NX; ++s) {
      const int ih = ih0[s] + dh_off, iw = iw0[s] + dw_off;
      const bool ok = kvalid && pvalid[s] && (unsigned)ih < (unsigned)a.ih &&
                      (unsigned)iw < (unsigned)a.iw;
      v4i v = {0, 0, 0, 0};
      if (ok)
        v = *reinterpret_cast<const v4i *>(a.x + xbase[s] +
                                           ((int64_t)ih * a.iw + iw) * a.x_cs + cgrp * 16);
      xreg[s] = v;
    }
    // advance to the next step's K group
    kg += 4;
    cgrp += 4;
    while (cgrp >= a.c16) {
      cgrp -= a.c16;
      if (++tkw == a.kw) {
        tkw = 0;
        ++tkh;
      }
    }
  };

  auto store_tile = [&](int buf) {
    v4i *base = lds[buf];
    if (wsmall) {
      if (lrow < BM) base[lrow * 4 + (kc ^ ((lrow >> 2) & 3))] = wreg[0];
    } else {
#pragma unroll
      for (int s = 0; s < NW; ++s) {
        const int r = lrow + 64 * s;
        base[r * 4 + (kc ^ ((r >> 2) & 3))] = wreg[s];
      }
    }
#pragma unroll
    for (int s = 0; s < NX; ++s) {
      const int r = lrow + 64 * s;
      base[(BM + r) * 4 + (kc ^ ((r >> 2) & 3))] = xreg[s];
    }
  };

  v16i acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

  const int nsteps = a.kp / 64;
  load_tile(0);
  store_tile(0);
  __syncthreads();

  const int frow = lane & 31;   // row inside a 32-row block
  const int fk = lane >> 5;     // which 16-byte half of a 32-byte MFMA K slice

  for (int step = 0; step < nsteps; ++step) {
    const int buf = step & 1;
    if (step + 1 < nsteps) load_tile(step + 1);
    const v4i *wl = lds[buf];
    const v4i *xl = lds[buf] + BM * 4;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const int chunk = kk * 2 + fk;
      v4i af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int r = (wm * TM + i) * 32 + frow;
        af[i] = wl[r * 4 + (chunk ^ ((r >> 2) & 3))];
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int r = (wn * TN + j) * 32 + frow;
        bf[j] = xl[r * 4 + (chunk ^ ((r >> 2) & 3))];
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i], bf[j], acc[i][j], 0, 0, 0);
    }
    if (step + 1 < nsteps) store_tile(buf ^ 1);
    __syncthreads();
  }

  // ---- epilogue.  In a 32x32 result block lane l holds column (pixel) l & 31
  // and rows (channels) 8*(r/4) + 4*(l/32) + r%4 for register r = 0..15, i.e.
  // four runs of 4 consecutive channels: each run becomes one 32-bit store.
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int pix = pix0 + (wn * TN + j) * 32 + frow;
    if (pix >= a.npix) continue;
    int8_t *yrow = a.y + (int64_t)pix * a.y_cs;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int oc = oc0 + (wm * TM + i) * 32 + q * 8 + fk * 4;
        if (oc >= a.ocw) continue;
        uint32_t word = 0;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int32_t v = epilogue(acc[i][j][q * 4 + b], a.cp[oc + b], a.lo, a.relu_first);
          word |= ((uint32_t)v & 0xffu) << (8 * b);
        }
        *reinterpret_cast<uint32_t *>(yrow + oc) = word;
      }
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
namespace {

struct TileCfg {
  int bm, bn;
};
const TileCfg kTiles[] = {{128, 128}, {64, 256}, {32, 256}};

int pick_tile(int ocp16) {
  if (ocp16 > 64) return 0;
  if (ocp16 > 32) return 1;
  return 2;
}

int check_desc(const tpuhip_conv_desc &d) {
  TPUHIP_REQUIRE(d.n > 0 && d.ic > 0 && d.ih > 0 && d.iw > 0 && d.oc > 0 && d.oh > 0 && d.ow > 0,
                 "conv: non-positive dimension");
  TPUHIP_REQUIRE(d.g > 0 && d.ic % d.g == 0 && d.oc % d.g == 0, "conv: bad group count %d", d.g);
  TPUHIP_REQUIRE(d.kh > 0 && d.kw > 0 && d.sh > 0 && d.sw > 0 && d.dh > 0 && d.dw > 0,
                 "conv: bad kernel/stride/dilation");
  TPUHIP_REQUIRE(d.pt >= 0 && d.pb >= 0 && d.pl >= 0 && d.pr >= 0 && d.ins_h >= 0 && d.ins_w >= 0,
                 "conv: negative padding");
  TPUHIP_REQUIRE(d.x_cs >= d.ic && d.y_cs >= d.oc && d.x_cs % 16 == 0 && d.y_cs % 16 == 0,
                 "conv: channel strides must be multiples of 16 covering the channels "
                 "(x_cs %d ic %d, y_cs %d oc %d)", d.x_cs, d.ic, d.y_cs, d.oc);
  const int ihd = (d.ih - 1) * (d.ins_h + 1) + 1, iwd = (d.iw - 1) * (d.ins_w + 1) + 1;
  const int oh = (ihd + d.pt + d.pb - (d.dh * (d.kh - 1) + 1)) / d.sh + 1;
  const int ow = (iwd + d.pl + d.pr - (d.dw * (d.kw - 1) + 1)) / d.sw + 1;
  // the reference's importers may round up (Caffe ceil mode) by padding b/r; all
  // that matters for memory safety is that every output maps to a legal window
  TPUHIP_REQUIRE(d.oh <= oh && d.ow <= ow, "conv: output %dx%d larger than the window grid %dx%d",
                 d.oh, d.ow, oh, ow);
  TPUHIP_REQUIRE((int64_t)d.n * d.oh * d.ow < (1ll << 31) &&
                     (int64_t)d.n * d.ih * d.iw * d.x_cs < (1ll << 40),
                 "conv: tensor too large");
  return TPUHIP_OK;
}

}  // namespace

extern "C" {

int tpuhip_conv2d_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *desc, const int8_t *filter,
                          const int32_t *bias, const int32_t *multiplier, const int32_t *rshift,
                          tpuhip_conv_weights **out) {
  TPUHIP_REQUIRE(ctx && desc && filter && multiplier && rshift && out,
                 "tpuhip_conv2d_prepack: NULL argument");
  const tpuhip_conv_desc &d = *desc;
  if (int rc = check_desc(d)) return rc;
  for (int i = 0; i < d.oc; ++i)
    TPUHIP_REQUIRE(rshift[i] >= 0 && rshift[i] <= 31, "conv: rshift[%d] = %d outside [0,31]", i,
                   rshift[i]);
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));

  const int icg = d.ic / d.g, ocg = d.oc / d.g;
  const bool dense = d.g == 1 && d.ins_h == 0 && d.ins_w == 0;
  const bool depthwise = d.g == d.ic && d.g == d.oc && d.ins_h == 0 && d.ins_w == 0;
  int algo = d.algo;
  if (algo == ALGO_AUTO) algo = dense ? ALGO_MFMA : depthwise ? ALGO_DEPTHWISE : ALGO_DIRECT;
  TPUHIP_REQUIRE(algo >= ALGO_DIRECT && algo <= ALGO_DEPTHWISE, "conv: unknown algo %d", d.algo);
  TPUHIP_REQUIRE(algo != ALGO_MFMA || dense, "conv: MFMA path needs g == 1 and no inserted zeros");
  TPUHIP_REQUIRE(algo != ALGO_DEPTHWISE || depthwise,
                 "conv: depthwise path needs g == ic == oc and no inserted zeros");

  auto *cw = new tpuhip_conv_weights();
  cw->d = d;
  cw->algo = algo;
  std::vector<int8_t> packed;
  if (algo == ALGO_MFMA) {
    cw->tile = pick_tile(round_up(d.oc, 16));
    const int bm = kTiles[cw->tile].bm;
    cw->ocp = round_up(d.oc, bm);
    const int icp = round_up(d.ic, 16);
    cw->c16 = icp / 16;
    cw->k16 = d.kh * d.kw * cw->c16;
    cw->kp = round_up(cw->k16 * 16, 64);
    packed.assign((size_t)cw->ocp * cw->kp, 0);
    for (int oc = 0; oc < d.oc; ++oc)
      for (int c = 0; c < d.ic; ++c)
        for (int kh = 0; kh < d.kh; ++kh)
          for (int kw = 0; kw < d.kw; ++kw)
            packed[(size_t)oc * cw->kp + (size_t)(kh * d.kw + kw) * icp + c] =
                filter[(((size_t)oc * d.ic + c) * d.kh + kh) * d.kw + kw];
  } else if (algo == ALGO_DEPTHWISE) {
    cw->ocp = round_up(d.oc, 16);
    packed.assign((size_t)d.kh * d.kw * cw->ocp, 0);
    for (int c = 0; c < d.oc; ++c)
      for (int kh = 0; kh < d.kh; ++kh)
        for (int kw = 0; kw < d.kw; ++kw)
          packed[(size_t)(kh * d.kw + kw) * cw->ocp + c] =
              filter[((size_t)c * d.kh + kh) * d.kw + kw];
  } else {
    cw->ocp = d.oc;
    packed.assign((size_t)d.oc * d.kh * d.kw * icg, 0);
    for (int oc = 0; oc < d.oc; ++oc)
      for (int c = 0; c < icg; ++c)
        for (int kh = 0; kh < d.kh; ++kh)
          for (int kw = 0; kw < d.kw; ++kw)
            packed[(((size_t)oc * d.kh + kh) * d.kw + kw) * icg + c] =
                filter[(((size_t)oc * icg + c) * d.kh + kh) * d.kw + kw];
  }
  (void)ocg;
  std::vector<ChanParams> cp((size_t)cw->ocp);
  for (int i = 0; i < cw->ocp; ++i) {
    ChanParams p{};
    if (i < d.oc) {
      p.bias = (d.with_bias && bias) ? bias[i] : 0;
      p.mult = multiplier[i];
      p.rshift = rshift[i];
      p.mask = (int32_t)((1ll << rshift[i]) - 1);
      p.half = p.mask >> 1;
    }
    cp[i] = p;
  }
  int rc = tpuhip_malloc(ctx, packed.size(), (void **)&cw->w);
  if (!rc) rc = tpuhip_malloc(ctx, cp.size() * sizeof(ChanParams), (void **)&cw->cp);
  if (!rc) rc = tpuhip_upload(ctx, cw->w, packed.data(), packed.size());
  if (!rc) rc = tpuhip_upload(ctx, cw->cp, cp.data(), cp.size() * sizeof(ChanParams));
  if (rc) {
    tpuhip_conv2d_weights_destroy(ctx, cw);
    return rc;
  }
  *out = cw;
  return TPUHIP_OK;
}

int tpuhip_conv2d_weights_destroy(tpuhip_ctx *ctx, tpuhip_conv_weights *w) {
  if (!w) return TPUHIP_OK;
  TPUHIP_REQUIRE(ctx, "tpuhip_conv2d_weights_destroy: NULL context");
  int rc = tpuhip_free(ctx, w->w);
  int rc2 = tpuhip_free(ctx, w->cp);
  delete w;
  return rc ? rc : rc2;
}

const char *tpuhip_conv2d_algo_name(const tpuhip_conv_weights *w) {
  if (!w) return "null";
  switch (w->algo) {
    case ALGO_DIRECT: return "direct";
    case ALGO_DEPTHWISE: return "depthwise";
    case ALGO_MFMA:
      return w->tile == 0 ? "mfma_128x128" : w->tile == 1 ? "mfma_64x256" : "mfma_32x256";
  }
  return "?";
}

int tpuhip_conv2d_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && w && x && y, "tpuhip_conv2d_i8: NULL argument");
  const tpuhip_conv_desc &d = w->d;
  ConvArgs a{};
  a.x = (const int8_t *)x;
  a.w = w->w;
  a.cp = w->cp;
  a.y = (int8_t *)y;
  a.n = d.n; a.ih = d.ih; a.iw = d.iw; a.x_cs = d.x_cs;
  a.oh = d.oh; a.ow = d.ow; a.y_cs = d.y_cs;
  a.oc = d.oc; a.ocw = round_up(d.oc, 16); a.icg = d.ic / d.g; a.ocg = d.oc / d.g; a.g = d.g;
  a.kh = d.kh; a.kw = d.kw; a.sh = d.sh; a.sw = d.sw; a.pt = d.pt; a.pl = d.pl;
  a.dh = d.dh; a.dw = d.dw; a.ins_h = d.ins_h; a.ins_w = d.ins_w;
  a.c16 = w->c16; a.k16 = w->k16; a.kp = w->kp;
  a.npix = d.n * d.oh * d.ow;
  a.lo = (d.do_relu && !d.relu_first) ? 0 : -128;
  a.relu_first = (d.do_relu && d.relu_first) ? 1 : 0;

  if (w->algo == ALGO_MFMA) {
    const TileCfg t = kTiles[w->tile];
    dim3 grid((unsigned)((a.npix + t.bn - 1) / t.bn), (unsigned)(w->ocp / t.bm));
    switch (w->tile) {
      case 0:
        hipLaunchKernelGGL((conv_mfma_kernel<128, 128, 2, 2>), grid, dim3(256), 0, ctx->stream, a);
        break;
      case 1:
        hipLaunchKernelGGL((conv_mfma_kernel<64, 256, 1, 4>), grid, dim3(256), 0, ctx->stream, a);
        break;
      default:
        hipLaunchKernelGGL((conv_mfma_kernel<32, 256, 1, 4>), grid, dim3(256), 0, ctx->stream, a);
        break;
    }
  } else if (w->algo == ALGO_DEPTHWISE) {
    const int64_t total = (int64_t)a.npix * (a.ocw / 16);
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(total, 256), 1 << 20);
    hipLaunchKernelGGL(conv_depthwise_kernel, dim3(blocks), dim3(256), 0, ctx->stream, a);
  } else {
    const int64_t total = (int64_t)a.npix * a.ocw;
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(total, 256), 1 << 20);
    hipLaunchKernelGGL(conv_direct_kernel, dim3(blocks), dim3(256), 0, ctx->stream, a);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_fc_prepack(tpuhip_ctx *ctx, int m, int k, int n, int x_cs, int y_cs, int do_relu,
                      const int8_t *filter_nk, const int32_t *bias, int32_t multiplier,
                      int32_t rshift, tpuhip_conv_weights **out) {
  TPUHIP_REQUIRE(m > 0 && k > 0 && n > 0, "fc: non-positive dimension");
  tpuhip_conv_desc d{};
  d.n = m; d.ic = k; d.ih = 1; d.iw = 1;
  d.oc = n; d.oh = 1; d.ow = 1;
  d.g = 1; d.kh = 1; d.kw = 1; d.sh = 1; d.sw = 1; d.dh = 1; d.dw = 1;
  d.do_relu = do_relu;
  d.with_bias = bias != nullptr;
  d.x_cs = x_cs; d.y_cs = y_cs;
  d.relu_first = 1;
  std::vector<int32_t> mult((size_t)n, multiplier), rs((size_t)n, rshift);
  return tpuhip_conv2d_prepack(ctx, &d, filter_nk, bias, mult.data(), rs.data(), out);
}

}  // extern "C"

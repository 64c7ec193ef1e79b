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
#include "conv_epilogue.hpp"

#include <map>
#include <mutex>

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <string>
#include <type_traits>
#include <vector>

using namespace tpuhip;


enum ConvAlgo { ALGO_AUTO = 0, ALGO_DIRECT = 1, ALGO_MFMA = 2, ALGO_DEPTHWISE = 3, ALGO_DEPTHWISE_DOT = 4,
                ALGO_STEM = 5 };

// per-channel requantisation record
struct __attribute__((aligned(16))) QParam {
  int32_t mult;
  int32_t rshift;
  int32_t mask;   // 2^rshift - 1
  int32_t hpot;   // 2^(rshift-1), 0 for rshift 0
};

struct tpuhip_conv_weights {
  tpuhip_conv_desc d;
  int algo = ALGO_DIRECT;
  int tile = 0;          // MFMA tile variant
  int fast = 0;          // the overflow-free requant form is provably exact for this layer
  bool smallc = false;   // ic <= 4: K packs 4 taps x 4 channels per 16-byte group (LDS kernels only)
  bool tuned = true;     // false: the tile is chosen by timing the candidates on first use
  // a pair of convs over one input packed as one: first channel, channel stride and ReLU of
  // the second result (split_oc == 0: an ordinary conv)
  int split_oc = 0, y2_cs = 0, relu2 = 0;
  // a FullyConnected whose K is beyond what the conv kernels index (more than 4096 input
  // channels): only the K-splitting FullyConnected kernels, which walk K linearly, run it
  bool fc_only = false;
  std::vector<int8_t> host_filter;  // OIHW copy, kept while the layer can still be repacked
  int8_t *w = nullptr;   // packed filter
  int32_t *bias = nullptr;
  QParam *qp = nullptr;
  int32_t *qplanes = nullptr;   // mult | rshift | hpot planes of nparam entries each
  int32_t *qc64 = nullptr;      // (low, high) pairs of bias * mult + 2^30, then the same + 2^(rshift-1) * 2^31
  int nparam = 0;
  int ocp = 0;           // padded output channels (rows of w / entries of bias, qp)
  int kp = 0;            // padded K in bytes (row stride of w) for the MFMA path
  int c16 = 0;           // input 16-channel groups per tap
  int k16 = 0;           // 16-byte K groups in total
};

struct ConvArgs {
  const int8_t *x;
  const int8_t *w;
  const int32_t *bias;
  const QParam *qp;
  const int32_t *qmult, *qshift, *qhpot;   // the same per-channel data as planes (MFMA epilogue)
  // per channel, as (low, high) word pairs: qc64 = bias * mult + 2^30, the addend of the
  // requantisation's 64-bit multiply-add; qc64r = qc64 + 2^(rshift-1) * 2^31, which also carries
  // the rounding term of the right shift (layers with a fused ReLU)
  const int32_t *qc64, *qc64r;
  int8_t *y;
  int n, ih, iw, x_cs;
  int oh, ow, y_cs;
  int oc, ocw, icg, ocg, g;  // ocw = oc rounded up to 16: channels written per pixel
  int kh, kw, sh, sw, pt, pl, dh, dw, ins_h, ins_w;
  int c16, k16, kp;
  uint32_t magic_c16, magic_kw;   // floor(2^20 / d) + 1: x / d == (x * magic) >> 20 for x < 4095
  uint32_t x_bytes, w_bytes;      // sizes behind x and w (buffer descriptors)
  uint32_t magic_ow, magic_oh;    // ceil(2^32 / d): x / d == umulhi(x, magic) for x, d < 2^16
  int n_oc_tiles, n_tiles, tiles_per_xcd;
  // ceil(2^32 / n_oc_tiles): tile / n_oc_tiles == umulhi(tile, magic) while tile * n_oc_tiles < 2^32;
  // 0 where there is nothing to divide by (one channel tile) or the product leaves that range
  uint32_t magic_oc_tiles;
  // persistent kernels: workgroups per XCD (a multiple of n_oc_tiles) and the pixel
  // advance between two tiles of one workgroup, split into (n, oh, ow) parts
  int wgs_per_xcd, pstep_pix, pstep_n, pstep_oh, pstep_ow;
  int tile_imgs;          // third form of the patch kernel: whole images per tile
  int npix;
  int linear;             // 1x1, stride 1, no padding: input pixel index == output pixel index
  int stem_pw;            // stem kernel: input columns one row tile needs, (128 - 1) * sw + 8
  uint32_t magic_pw;      // floor(2^20 / stem_pw) + 1
  int lo;          // lower clamp bound: 0 with ReLU after saturation, else -128
  int relu_first;  // ReLU on the sum before requantisation (FC)
  // optional fused eltwise add on the conv result (same shape and channel stride as y):
  // add_dst = sat8(floor(relu?(add_src * add_m_src + y * add_m_conv) / 2^add_rshift + 0.5))
  const int8_t *add_src;
  int8_t *add_dst;
  int add_m_src, add_m_conv, add_rshift, add_relu;
  int add_pk;      // |multipliers| <= 127 and rshift <= 8: the sum fits packed int16 arithmetic
  int store_y;     // 0: the conv result itself is not written (only what is fused behind it)
  // two convolutions over one input run as one (their filters stacked along oc): channels
  // from split_oc on (a multiple of 128, 0 = no second conv) belong to the second one and
  // go to y2 with its own channel stride and ReLU
  int split_oc, y2_cs, lo2;
  int8_t *y2;
  // optional fused 256-entry table on the conv result, applied before the fused add:
  // lut_dst (may be null) receives table[y]; the add then takes table[y]
  int has_lut;
  int8_t *lut_dst;
  Table256 lut;
#ifdef TPUHIP_TRACE
  unsigned long long *trace;   // development builds: 32 shader-clock stamps per workgroup
#endif
};
#ifdef TPUHIP_TRACE
#define TPUHIP_TS(k) (ts[k] = (unsigned long long)clock64())
#else
#define TPUHIP_TS(k) ((void)0)
#endif

__device__ __forceinline__ int32_t epilogue(int32_t acc, int32_t bias, const QParam &p, int lo,
                                            int relu_first) {
  int32_t v = (int32_t)((uint32_t)acc + (uint32_t)bias);
  if (relu_first) v = max(v, 0);
  return requant_qdm(v, p.mult, p.rshift, p.mask, p.mask >> 1, lo);
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
    *yp = (int8_t)epilogue(acc, a.bias[oc], a.qp[oc], a.lo, a.relu_first);
  }
}

__device__ __forceinline__ int32_t sbyte(int32_t word, int i) {
  return (int32_t)(int8_t)(word >> (8 * i));
}

// ---------------------------------------------------------------------------
// MFMA implicit-GEMM kernel.
//
//   D[oc][pix] = sum_k W[oc][k] * X[pix][k],   k = (kh*KW + kw)*icp + c
//
// (icp = input channels rounded up to 16).  A workgroup of WM x WN waves owns a
// tile of BM output channels x BN pixels; every wave owns (BM/WM) x (BN/WN) of it
// as TM x TN blocks of 32x32 (v_mfma_i32_32x32x32_i8).  K is consumed BK bytes per
// step.  Global loads run DEPTH steps ahead of the MFMAs in a ring of registers,
// LDS is double-buffered, one barrier per step.
//
// LDS rows are BK bytes (BK/16 chunks of 16); the chunk index is XOR-swizzled with
// row bits chosen so that 16 consecutive rows of one chunk cover 256 distinct
// bytes of bank space, for the loader's 16-byte stores and the fragment reads alike.
//
// The rows of a weight tile are stored permuted (see mfma_row_to_oc) so that in
// the 32x32 result layout -- lane l holds column l & 31 and rows
// 8*(r/4) + 4*(l/32) + r%4 for register r -- the 16 registers of a lane are 16
// consecutive output channels of one pixel: one 16-byte store per block.
// ---------------------------------------------------------------------------

// FAST: every channel has 1 <= rshift <= 31 and |acc + bias| + 1 + 2^(rshift-1) < 2^31
// (proved on the host from the weights), so RoundingDivideByPOT is
// (x + 2^(e-1) - (x < 0)) >> e without overflow.
template <bool FAST>
__device__ __forceinline__ int32_t requant_core(int32_t v, int32_t mult, int32_t rshift,
                                                int32_t hpot) {
  const int32_t x = srdhm(v, mult);
  if (FAST) return (x + hpot + (x >> 31)) >> rshift;
  const int32_t mask = (int32_t)((1u << rshift) - 1u);   // rshift <= 31
  return rdbp(x, rshift, mask, mask >> 1);
}

// Where an output-channel tile is written.  A pair of convs packed as one: a workgroup (or
// wave) whose tile lies in the second conv's channels writes that conv's result, with its
// channel stride and ReLU; split_oc is a multiple of 128, so no tile straddles it.  Chosen
// once per workgroup, before any tile is computed, from a uniform tile base.
struct OutRoute {
  int8_t *y;
  int y_cs, lo, shift;   // shift: first channel of the tensor written
};
__device__ __forceinline__ OutRoute route_out(const ConvArgs &a, int oc_tile_base) {
  const bool second = a.split_oc > 0 && oc_tile_base >= a.split_oc;
  return OutRoute{second ? a.y2 : a.y, second ? a.y2_cs : a.y_cs, second ? a.lo2 : a.lo,
                  second ? a.split_oc : 0};
}

// Requantises the lane's 16 consecutive channels of TN pixels (one row block of a wave tile):
// saturated (+ReLU) bytes, 16 per pixel.  Parameters are read four channels at a time to keep
// few registers live.
template <int TN, bool FAST>
__device__ __forceinline__ void requant_rows(const v16i (&acc)[TN], int relu_first, int lo,
                                             const int32_t *pmult, const int32_t *pshift,
                                             const int32_t *phpot, uint32_t (&outw)[TN][4]) {
#pragma unroll
  for (int qd = 0; qd < 4; ++qd) {
    const v4i m4 = *reinterpret_cast<const v4i *>(pmult + qd * 4);
    const v4i r4 = *reinterpret_cast<const v4i *>(pshift + qd * 4);
    const v4i h4 = *reinterpret_cast<const v4i *>(phpot + qd * 4);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      int32_t v0 = acc[j][qd * 4 + 0], v1 = acc[j][qd * 4 + 1], v2 = acc[j][qd * 4 + 2],
              v3 = acc[j][qd * 4 + 3];
      if (relu_first) {
        v0 = max(v0, 0); v1 = max(v1, 0); v2 = max(v2, 0); v3 = max(v3, 0);
      }
      outw[j][qd] = pack_sat4(requant_core<FAST>(v0, m4[0], r4[0], h4[0]),
                              requant_core<FAST>(v1, m4[1], r4[1], h4[1]),
                              requant_core<FAST>(v2, m4[2], r4[2], h4[2]),
                              requant_core<FAST>(v3, m4[3], r4[3], h4[3]), lo);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
}

// What happens to 16 requantised channels (first channel oc of the launch, byte offset off in
// the tensor written): the store, the fused table, the fused add with its operand sv.
__device__ __forceinline__ void finish_chunk(v4i o, const v4i &sv, int64_t off, int oc, const ConvArgs &a,
                                             int8_t *ydst, const uint8_t *lut) {
  if (a.store_y) *reinterpret_cast<v4i *>(ydst + off) = o;
  if (lut) {
    // table lookup per byte (index = the two's-complement byte); the 256-byte table
    // covers each LDS bank once, so any 64 indices are conflict-free.  Pad channels
    // stay zero whatever table[0] is.
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const uint32_t wd = (uint32_t)o[q];
      const uint32_t r = (uint32_t)lut[wd & 255u] | ((uint32_t)lut[(wd >> 8) & 255u] << 8) |
                         ((uint32_t)lut[(wd >> 16) & 255u] << 16) | ((uint32_t)lut[wd >> 24] << 24);
      const int valid = a.oc - (oc + q * 4);   // channels of this dword that exist
      const uint32_t mask = valid >= 4 ? 0xffffffffu : valid <= 0 ? 0u : (1u << (8 * valid)) - 1u;
      o[q] = (int)(r & mask);
    }
    if (a.lut_dst) *reinterpret_cast<v4i *>(a.lut_dst + off) = o;
  }
  if (a.add_dst)
    *reinterpret_cast<v4i *>(a.add_dst + off) =
        fused_add_chunk(o, sv, a.add_m_src, a.add_m_conv, a.add_rshift, a.add_relu, a.add_pk);
}

// Epilogue of one wave tile row block, written straight from the MFMA result layout: every
// lane stores the 16 bytes of its own pixel.
// pix_limit: pixels from this index on are not written (a.npix, or the end of a tile that
// stops short of its 32-pixel blocks)
template <int TN, bool FAST>
__device__ __forceinline__ void epilogue_rows_lim(const v16i (&acc)[TN], const ConvArgs &a, int oc,
                                                  const int32_t *pmult, const int32_t *pshift,
                                                  const int32_t *phpot, int pix_first, int pix_stride,
                                                  const uint8_t *lut, const OutRoute &out, int pix_limit) {
  uint32_t outw[TN][4];
  // channel index within the tensor written (a pair's second result starts at split_oc)
  const int ycs = out.y_cs;
  const int ocl = oc - out.shift;
  // the other operand of a fused add is fetched now and used after the requantisation
  v4i sv[TN];
  if (a.add_dst) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int pix = min(pix_first + j * pix_stride, a.npix - 1);
      sv[j] = *reinterpret_cast<const v4i *>(a.add_src + (int64_t)pix * ycs + ocl);
    }
  }
  requant_rows<TN, FAST>(acc, a.relu_first, out.lo, pmult, pshift, phpot, outw);
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int pix = pix_first + j * pix_stride;
    if (pix < pix_limit) {
      const v4i o = {(int)outw[j][0], (int)outw[j][1], (int)outw[j][2], (int)outw[j][3]};
      finish_chunk(o, sv[j], (int64_t)pix * ycs + ocl, oc, a, out.y, lut);
    }
  }
}

// The same epilogue through LDS, so that global memory sees whole rows: a workgroup's tile of
// BM channels x BN pixels is requantised into a staging area (stage_rows: rows of BM bytes +
// 16 bytes of padding, which spreads the 16-byte writes of 8 neighbouring pixels over all
// banks), and after a barrier the threads walk it in memory order -- BM / 16 neighbouring
// lanes cover one pixel's BM contiguous bytes -- doing the fused table / add and the stores
// there.  A lane-per-pixel store touches 64 different lines per instruction; written this way
// a 256-byte-row tensor takes a third of the time.
template <int BM>
constexpr int stage_row_bytes() { return BM + 16; }

template <int TM, int TN, int BM, bool FAST>
__device__ __forceinline__ void stage_rows(const v16i (&acc)[TM][TN], int relu_first, int lo, int8_t *stage,
                                           int row0, int col0, const int32_t *pmult, const int32_t *pshift,
                                           const int32_t *phpot) {
  // row0: the lane's first pixel row in the tile (rows j * 32 further on follow), col0: its
  // first channel byte; the parameter pointers are those of col0
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    uint32_t outw[TN][4];
    requant_rows<TN, FAST>(acc[i], relu_first, lo, pmult + i * 16, pshift + i * 16, phpot + i * 16, outw);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      *reinterpret_cast<v4i *>(stage + (row0 + j * 32) * stage_row_bytes<BM>() + col0 + i * 16) =
          v4i{(int)outw[j][0], (int)outw[j][1], (int)outw[j][2], (int)outw[j][3]};
  }
}

// chunks of 16 bytes of a BM x BN tile handled per thread
template <int BM, int BN, int NT>
constexpr int flush_chunks() { return (BN * (BM / 16) + NT - 1) / NT; }

// requests the fused add's other operand for this thread's chunks (before the requantisation,
// whose arithmetic then hides the latency)
template <int BM, int BN, int NT>
__device__ __forceinline__ void flush_prefetch(const ConvArgs &a, int tid, int pix0, int pix_limit, int oc0,
                                               const OutRoute &out, v4i (&sv)[flush_chunks<BM, BN, NT>()]) {
  constexpr int CPR = BM / 16, NU = flush_chunks<BM, BN, NT>();
  if (!a.add_dst) return;
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int q = tid + u * NT;
    const int row = q / CPR, cc = q - row * CPR;
    const int pix = pix0 + row, oc = oc0 + cc * 16;
    if (q < BN * CPR && pix < pix_limit && oc < a.ocw)
      sv[u] = *reinterpret_cast<const v4i *>(a.add_src + (int64_t)pix * out.y_cs + (oc - out.shift));
  }
}

template <int BM, int BN, int NT>
__device__ __forceinline__ void flush_tile(const ConvArgs &a, const int8_t *stage, int tid, int pix0,
                                           int pix_limit, int oc0, const OutRoute &out, const uint8_t *lut,
                                           const v4i (&sv)[flush_chunks<BM, BN, NT>()]) {
  constexpr int CPR = BM / 16, NU = flush_chunks<BM, BN, NT>();
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int q = tid + u * NT;
    const int row = q / CPR, cc = q - row * CPR;
    const int pix = pix0 + row, oc = oc0 + cc * 16;
    if (q < BN * CPR && pix < pix_limit && oc < a.ocw) {
      const v4i o = *reinterpret_cast<const v4i *>(stage + row * stage_row_bytes<BM>() + cc * 16);
      finish_chunk(o, sv[u], (int64_t)pix * out.y_cs + (oc - out.shift), oc, a, out.y, lut);
    }
  }
}

template <int TN, bool FAST>
__device__ __forceinline__ void epilogue_rows(const v16i (&acc)[TN], const ConvArgs &a, int oc,
                                              const int32_t *pmult, const int32_t *pshift,
                                              const int32_t *phpot, int pix_first,
                                              int pix_stride, const uint8_t *lut, const OutRoute &out) {
  epilogue_rows_lim<TN, FAST>(acc, a, oc, pmult, pshift, phpot, pix_first, pix_stride, lut, out, a.npix);
}


// how a K group maps to filter taps (see load_tile)
constexpr int kModeGeneral = 0;   // per-lane tap arithmetic
constexpr int kModeUniform = 1;   // ic % (BK) == 0: all groups of a step in one tap, scalar arithmetic
constexpr int kModeSmallC = 2;    // ic <= 4: four taps per 16-byte group


// The kernel arguments (ConvArgs: six 64-byte lines before the table) arrive through the scalar
// cache.  The compiler fetches a field where it first needs it, and what lies between kernel entry
// and a layer's first load needs some thirty of them: a dozen and more scalar loads, each with its
// own wait, one after the other (the first to touch a line a miss), before the first address of
// the layer is known.  Naming them all as inputs of one (empty) asm statement makes them due at
// one point: the loads go out together, merged where the fields are neighbours, behind a single
// wait.
__device__ __forceinline__ void gather_conv_args(const ConvArgs &a) {
  asm volatile("" ::"s"(a.x), "s"(a.w), "s"(a.bias), "s"(a.qmult), "s"(a.qshift), "s"(a.qhpot), "s"(a.y), "s"(a.x_bytes),
               "s"(a.w_bytes), "s"(a.tiles_per_xcd), "s"(a.n_tiles), "s"(a.n_oc_tiles), "s"(a.linear), "s"(a.x_cs),
               "s"(a.npix), "s"(a.kp), "s"(a.c16), "s"(a.k16), "s"(a.has_lut), "s"(a.wgs_per_xcd), "s"(a.ow), "s"(a.oh),
               "s"(a.ih), "s"(a.iw), "s"(a.sh), "s"(a.sw), "s"(a.pt), "s"(a.pl), "s"(a.magic_c16), "s"(a.magic_kw));
}
// tile index -> pixel tile (the channel tile is the remainder): a multiply where the host could
// give its constant, the generic division otherwise
__device__ __forceinline__ int pixel_tile_of(const ConvArgs &a, int tile) {
  if (a.n_oc_tiles == 1) return tile;
  if (a.magic_oc_tiles) return (int)__umulhi((uint32_t)tile, a.magic_oc_tiles);
  return tile / a.n_oc_tiles;
}

// the second list: what the LDS kernels' tile walk and epilogue set-up read as well
__device__ __forceinline__ void gather_conv_args_more(const ConvArgs &a) {
  asm volatile("" ::"s"(a.magic_oc_tiles), "s"(a.split_oc), "s"(a.magic_ow), "s"(a.magic_oh), "s"(a.pstep_pix), "s"(a.stem_pw), "s"(a.lo),
               "s"(a.ocw), "s"(a.qc64), "s"(a.qc64r), "s"(a.y_cs), "s"(a.store_y), "s"(a.add_dst), "s"(a.relu_first),
               "s"(a.magic_pw), "s"(a.dh), "s"(a.dw), "s"(a.kh), "s"(a.kw));
}

// ---------------------------------------------------------------------------
// depthwise kernel (g == ic == oc).  A lane owns 16 channels and walks pixels with a
// fixed stride, so its filter taps and requant parameters stay in registers.  The
// multiply-adds run as 4 x int8 dot products over FOUR TAPS of one channel: the four
// 16-byte loads of a tap group are byte-transposed (8 v_perm per 4 channels) into one
// dword per channel, and the filter is stored the same way, [tap group][channel] ->
// 4 taps.  Taps outside the image read zeros through the buffer descriptor.
// G = tap groups held in registers (kh*kw <= 4*G); G == 0 streams the filter instead.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void transpose4x4_bytes(uint32_t t0, uint32_t t1, uint32_t t2,
                                                   uint32_t t3, uint32_t (&c)[4]) {
  const uint32_t ab_lo = __builtin_amdgcn_perm(t1, t0, 0x05010400u);   // a0 b0 a1 b1
  const uint32_t ab_hi = __builtin_amdgcn_perm(t1, t0, 0x07030602u);   // a2 b2 a3 b3
  const uint32_t cd_lo = __builtin_amdgcn_perm(t3, t2, 0x05010400u);
  const uint32_t cd_hi = __builtin_amdgcn_perm(t3, t2, 0x07030602u);
  c[0] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u);             // a0 b0 c0 d0
  c[1] = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
  c[2] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u);
  c[3] = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
}

template <int G, bool FAST>
__global__ __launch_bounds__(256) void conv_depthwise_kernel(ConvArgs a) {
  __shared__ uint32_t lutw[64];
  if (a.has_lut) {
    if (threadIdx.x < 64) lutw[threadIdx.x] = a.lut.w[threadIdx.x];
    __syncthreads();
  }
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  const int c16 = a.ocw >> 4;
  const int64_t gid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int nslots = (int)(((int64_t)gridDim.x * blockDim.x) / c16);   // pixels in flight
  const int cg = (int)(gid % c16);
  int pix = (int)(gid / c16);
  if (pix >= nslots) return;
  const int groups = (a.kh * a.kw + 3) >> 2;
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);

  // per-channel constants of this lane's 16 channels
  v4i wq[G > 0 ? G : 1][4], bias4[4], mult4[4], shift4[4];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    bias4[q] = *reinterpret_cast<const v4i *>(a.bias + cg * 16 + q * 4);
    mult4[q] = *reinterpret_cast<const v4i *>(a.qmult + cg * 16 + q * 4);
    shift4[q] = *reinterpret_cast<const v4i *>(a.qshift + cg * 16 + q * 4);
#pragma unroll
    for (int g = 0; g < G; ++g)
      wq[g][q] = *reinterpret_cast<const v4i *>(a.w + ((int64_t)g * a.ocw + cg * 16 + q * 4) * 4);
  }

  // (n, oh, ow) of the lane's pixel, advanced by the walk's stride with carries
  int ow = pix % a.ow;
  int oh = (pix / a.ow) % a.oh;
  int n = pix / (a.ow * a.oh);
  const int d_ow = nslots % a.ow, d_oh = (nslots / a.ow) % a.oh, d_n = nslots / (a.ow * a.oh);

  for (; pix < a.npix; pix += nslots) {
    const int ihb = oh * a.sh - a.pt, iwb = ow * a.sw - a.pl;
    const int base = ((n * a.ih + ihb) * a.iw + iwb) * a.x_cs + cg * 16;
    int32_t acc[16];
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[q * 4 + i] = bias4[q][i];
    auto tap_group = [&](int g, const v4i (&wg)[4]) {
      v4i t[4];
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const uint32_t tap = (uint32_t)(g * 4 + k);
        const int tkh = (int)((tap * a.magic_kw) >> 20);
        const int tkw = (int)tap - tkh * a.kw;
        const int ih = ihb + tkh * a.dh, iw = iwb + tkw * a.dw;
        const bool ok = ((int)tap < a.kh * a.kw) & ((unsigned)ih < (unsigned)a.ih) &
                        ((unsigned)iw < (unsigned)a.iw);
        t[k] = buffer_load16(xrsrc, ok ? (uint32_t)(base + (tkh * a.dh * a.iw + tkw * a.dw) * a.x_cs)
                                       : kOobOffset);
      }
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint32_t c[4];
        transpose4x4_bytes((uint32_t)t[0][q], (uint32_t)t[1][q], (uint32_t)t[2][q], (uint32_t)t[3][q], c);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          acc[q * 4 + i] = __builtin_amdgcn_sdot4((int)c[i], wg[q][i], acc[q * 4 + i], false);
      }
    };
    if (G > 0) {
#pragma unroll
      for (int g = 0; g < G; ++g) tap_group(g, wq[g]);
    } else {
      for (int g = 0; g < groups; ++g) {
        v4i wg[4];
#pragma unroll
        for (int q = 0; q < 4; ++q)
          wg[q] = *reinterpret_cast<const v4i *>(a.w + ((int64_t)g * a.ocw + cg * 16 + q * 4) * 4);
        tap_group(g, wg);
      }
    }
    v4i o;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      int32_t r[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        int32_t v = acc[q * 4 + i];
        if (a.relu_first) v = max(v, 0);
        const int32_t e = shift4[q][i];
        r[i] = requant_core<FAST>(v, mult4[q][i], e, (int32_t)((1u << e) >> 1));
      }
      o[q] = (int)pack_sat4(r[0], r[1], r[2], r[3], a.lo);
    }
    const int64_t off = (int64_t)pix * a.y_cs + cg * 16;
    if (a.store_y) *reinterpret_cast<v4i *>(a.y + off) = o;
    if (lut) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t wd = (uint32_t)o[q];
        const uint32_t r = (uint32_t)lut[wd & 255u] | ((uint32_t)lut[(wd >> 8) & 255u] << 8) |
                           ((uint32_t)lut[(wd >> 16) & 255u] << 16) | ((uint32_t)lut[wd >> 24] << 24);
        const int valid = a.oc - (cg * 16 + q * 4);
        const uint32_t mask = valid >= 4 ? 0xffffffffu : valid <= 0 ? 0u : (1u << (8 * valid)) - 1u;
        o[q] = (int)(r & mask);
      }
      if (a.lut_dst) *reinterpret_cast<v4i *>(a.lut_dst + off) = o;
    }
    ow += d_ow;
    if (ow >= a.ow) { ow -= a.ow; ++oh; }
    oh += d_oh;
    if (oh >= a.oh) { oh -= a.oh; ++n; }
    n += d_n;
  }
}


// UNI: the input channel count is a multiple of 64, so the four 16-byte K groups of
// a step lie in one filter tap and all tap arithmetic is wave-uniform (scalar).
// OCC: waves per SIMD the register allocation must allow (0 = whatever it takes).
// PERSIST: a workgroup walks several pixel tiles of one output-channel tile.  The
// launch holds about as many workgroups as fit on the chip at once; the requant
// parameters of the channel tile sit in LDS, and the first K tiles of the next
// pixel tile are fetched before the epilogue of the current one, so the global
// latency at the head of a tile hides behind the VALU work at the tail of the last.
template <int BM, int BN, int WM, int WN, int BK, int DEPTH, int OCC, bool PERSIST, bool FAST,
          int MODE>
__global__ __launch_bounds__(WM *WN * 64) __attribute__((amdgpu_waves_per_eu(OCC > 0 ? OCC : 1))) void
conv_mfma_kernel(ConvArgs a) {
#ifdef TPUHIP_TRACE
  unsigned long long ts[32] = {};
  bool first_tile = true;
#endif
  TPUHIP_TS(0);
  gather_conv_args(a);
  gather_conv_args_more(a);
  constexpr bool UNI = MODE == kModeUniform;
  constexpr bool SMALLC = MODE == kModeSmallC;
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32;  // 32x32 blocks per wave along oc
  constexpr int TN = BN / WN / 32;  // 32x32 blocks per wave along pixels
  static_assert(TM >= 1 && TN >= 1 && TM * WM * 32 == BM && TN * WN * 32 == BN, "bad tile");
  constexpr int CH = BK / 16;                // 16-byte chunks per tile row (K bytes per step / 16)
  constexpr int SW = CH == 4 ? 2 : CH == 8 ? 1 : 0;   // swizzle: chunk ^= (row >> SW) & (CH - 1)
  static_assert(BK == 64 || BK == 128 || BK == 256, "K bytes per step");
  constexpr int RP = NT / CH;                // tile rows fetched per pass of the workgroup
  constexpr int NW = (BM + RP - 1) / RP;     // 16-byte weight chunks per thread per step
  constexpr int NX = BN / RP;                // 16-byte activation chunks per thread per step
  static_assert(BN % RP == 0, "pixel tile must be a multiple of the loader pass");
  static_assert(DEPTH % 2 == 0 && DEPTH >= 2 && DEPTH <= 12, "register ring depth");

  __shared__ v4i lds[2][(BM + BN) * CH];
  // bias | multiplier | rshift | 2^(rshift-1) of the workgroup's BM channels
  __shared__ __attribute__((aligned(16))) int32_t qlds[PERSIST ? 4 * BM : 4];
  __shared__ uint32_t lutw[64];   // fused table (published by the first barrier of the K loop)

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // Workgroups are handed to the 8 XCDs round-robin; give each XCD a contiguous run
  // of tiles, output-channel tiles of one pixel tile next to each other, so that the
  // workgroups sharing activations (and writing the same output rows) share an L2.
  int ltile = (int)(blockIdx.x >> 3);                                   // tile index inside the XCD's run
  int logical = (int)(blockIdx.x & 7) * a.tiles_per_xcd + ltile;
  if (logical >= a.n_tiles) return;
  const int pix_tile = pixel_tile_of(a, logical);
  const int oc0 = (logical - pix_tile * a.n_oc_tiles) * BM;   // the same for every tile of a walk
  const OutRoute out = route_out(a, __builtin_amdgcn_readfirstlane(oc0));
  int pix0 = pix_tile * BN;

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

  // the fused table and the requant parameters of the channel tile: fetched now, parked in LDS
  // after the first tile loads have been issued (their latencies overlap instead of adding up)
  uint32_t lutv = 0;
  if (a.has_lut && tid < 64) lutv = a.lut.w[tid];
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  static_assert(!PERSIST || BM <= NT, "one parameter row per thread");
  int32_t qv[4] = {0, 0, 0, 0};
  if (PERSIST && tid < BM) {
    qv[0] = a.bias[oc0 + tid];
    qv[1] = a.qmult[oc0 + tid];
    qv[2] = a.qshift[oc0 + tid];
    qv[3] = a.qhpot[oc0 + tid];
  }

  // ---- loader state: this thread fetches K-chunk kc of rows lrow + RP*s
  const int kc = tid % CH;
  const int lrow = tid / CH;
  int poff[NX];     // byte offset of (n, oh*sh - pt, ow*sw - pl, kc*16) in x (may lie before the image)
  int ih0[NX], iw0[NX];
  // (n, oh, ow) of the tile's first pixel: one generic division per workgroup ...
  // (a 1x1 / stride 1 / unpadded conv reads the input pixel of the same index as the output
  // pixel: no coordinates at all, which takes three divisions and the per-row arithmetic out of
  // the path to the first load)
  int ow_first = 0, oh_first = 0, n_first = 0;
  if (!a.linear) {
    ow_first = pix0 % a.ow;
    const int t_first = pix0 / a.ow;
    oh_first = t_first % a.oh;
    n_first = t_first / a.oh;
  }
  auto setup_rows = [&]() {
    if (a.linear) {
#pragma unroll
      for (int s = 0; s < NX; ++s) {
        const int pix = pix0 + lrow + RP * s;
        ih0[s] = pix < a.npix ? 0 : -(1 << 28);
        iw0[s] = 0;
        poff[s] = pix * a.x_cs + (UNI ? kc * 16 : 0);
        asm volatile("" : "+v"(poff[s]), "+v"(ih0[s]), "+v"(iw0[s]));
      }
      return;
    }
#pragma unroll
    for (int s = 0; s < NX; ++s) {
      // ... and exact multiply-high divisions of small numbers per row
      const int delta = lrow + RP * s;
      const bool pv = pix0 + delta < a.npix;
      const uint32_t t1 = (uint32_t)(ow_first + delta);
      const uint32_t q1 = a.ow == 1 ? t1 : __umulhi(t1, a.magic_ow);
      const int ow = (int)(t1 - q1 * (uint32_t)a.ow);
      const uint32_t t2 = (uint32_t)oh_first + q1;
      const uint32_t q2 = a.oh == 1 ? t2 : __umulhi(t2, a.magic_oh);
      const int oh = (int)(t2 - q2 * (uint32_t)a.oh);
      const int n = n_first + (int)q2;
      ih0[s] = pv ? oh * a.sh - a.pt : -(1 << 28);   // an invalid pixel never passes the bounds test
      iw0[s] = ow * a.sw - a.pl;
      // (the product is pinned before the chunk offset is added: left to itself the compiler forms a
      // 64-bit multiply-add whose upper addend register is undefined, picks one that a parameter
      // load above is still due to write, and waits for that load before the first tile load is
      // issued -- a trip to memory for a value nobody reads)
      int pixel_bytes = ((n * a.ih + (oh * a.sh - a.pt)) * a.iw + iw0[s]) * a.x_cs;
      asm volatile("" : "+v"(pixel_bytes));
      poff[s] = pixel_bytes + (UNI ? kc * 16 : 0);
      // keep the three values in registers instead of recomputing them every K step
      asm volatile("" : "+v"(poff[s]), "+v"(ih0[s]), "+v"(iw0[s]));
    }
  };
  setup_rows();
  uint32_t woff[NW];
#pragma unroll
  for (int s = 0; s < NW; ++s) {
    const int r = lrow + RP * s;
    woff[s] = r < BM ? (uint32_t)((oc0 + r) * a.kp + kc * 16) : kOobOffset;
    asm volatile("" : "+v"(woff[s]));
  }

  v4i wreg[DEPTH][NW], xreg[DEPTH][NX];
  const int nsteps = a.kp / BK;

  // fetch the tile of K step `step` into ring slot `slot`; no branches, no state.
  // A 16-byte K group kg = tap * c16 + cgrp with tap = tkh * kw + tkw; the divisions
  // are exact multiply-shifts.
  auto load_tile = [&](int slot, int step) {
    const bool in_k = step < nsteps;
#pragma unroll
    for (int s = 0; s < NW; ++s)
      wreg[slot][s] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
          wrsrc, in_k ? woff[s] : kOobOffset, step * BK, 0);
    if (SMALLC) {
      // at most 4 input channels: a 16-byte K group is 4 filter taps x 4 channels, each
      // tap one dword of its own pixel (K index = tap * 4 + c)
      const int taps = a.kh * a.kw;
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t tap = (uint32_t)((step * CH + kc) * 4 + t);
        const int tkh = (int)((tap * a.magic_kw) >> 20);
        const int tkw = (int)tap - tkh * a.kw;
        const int dh_off = (int)tap < taps ? tkh * a.dh : (1 << 28);
        const int dw_off = tkw * a.dw;
        const int tap_off = (dh_off * a.iw + dw_off) * a.x_cs;
#pragma unroll
        for (int s = 0; s < NX; ++s) {
          const int ih = ih0[s] + dh_off, iw = iw0[s] + dw_off;
          const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
          xreg[slot][s][t] = (int)__builtin_amdgcn_raw_buffer_load_b32(
              xrsrc, ok ? (uint32_t)(poff[s] + tap_off) : kOobOffset, 0, 0);
        }
      }
    } else if (UNI) {
      const uint32_t kg0 = (uint32_t)(step * CH);
      const uint32_t tap = (kg0 * a.magic_c16) >> 20;
      const int cgrp0 = (int)(kg0 - tap * (uint32_t)a.c16);
      const int tkh = (int)((tap * a.magic_kw) >> 20);
      const int tkw = (int)tap - tkh * a.kw;
      // past the end of K the row offset is pushed out of every image
      const int dh_off = (int)kg0 < a.k16 ? tkh * a.dh : (1 << 28);
      const int dw_off = tkw * a.dw;
      const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp0 * 16;
#pragma unroll
      for (int s = 0; s < NX; ++s) {
        const int ih = ih0[s] + dh_off, iw = iw0[s] + dw_off;
        const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
        xreg[slot][s] = buffer_load16(xrsrc, ok ? (uint32_t)(poff[s] + tap_off) : kOobOffset);
      }
    } else {
      const uint32_t kg = (uint32_t)(step * CH + kc);
      const uint32_t tap = (kg * a.magic_c16) >> 20;
      const int cgrp = (int)(kg - tap * (uint32_t)a.c16);
      const int tkh = (int)((tap * a.magic_kw) >> 20);
      const int tkw = (int)tap - tkh * a.kw;
      const int dh_off = (int)kg < a.k16 ? tkh * a.dh : (1 << 28);
      const int dw_off = tkw * a.dw;
      const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp * 16;
#pragma unroll
      for (int s = 0; s < NX; ++s) {
        const int ih = ih0[s] + dh_off, iw = iw0[s] + dw_off;
        const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
        xreg[slot][s] = buffer_load16(xrsrc, ok ? (uint32_t)(poff[s] + tap_off) : kOobOffset);
      }
    }
  };

  auto store_tile = [&](int slot, int buf) {
    v4i *base = lds[buf];
#pragma unroll
    for (int s = 0; s < NW; ++s) {
      const int r = lrow + RP * s;
      if (BM % RP == 0 || r < BM) base[r * CH + (kc ^ ((r >> SW) & (CH - 1)))] = wreg[slot][s];
    }
#pragma unroll
    for (int s = 0; s < NX; ++s) {
      const int r = lrow + RP * s;
      base[(BM + r) * CH + (kc ^ ((r >> SW) & (CH - 1)))] = xreg[slot][s];
    }
  };

  const int frow = lane & 31;   // row inside a 32-row block
  const int fk = lane >> 5;     // which 16-byte half of a 32-byte MFMA K slice
  const int lch0 = wm * TM * 32 + fk * 16 * TM;   // first of this lane's 16*TM channels in the tile
  const int ocw0 = oc0 + lch0;

  v16i acc[TM][TN];
  constexpr int KK = BK / 32;
  v4i fa[2][TM], fb[2][TN];
  auto read_frag = [&](int buf, int kk, int fs) {
    const v4i *wl = lds[buf];
    const v4i *xl = lds[buf] + BM * CH;
    const int chunk = kk * 2 + fk;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r = (wm * TM + i) * 32 + frow;
      fa[fs][i] = wl[r * CH + (chunk ^ ((r >> SW) & (CH - 1)))];
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int r = (wn * TN + j) * 32 + frow;
      fb[fs][j] = xl[r * CH + (chunk ^ ((r >> SW) & (CH - 1)))];
    }
  };
  auto mfma_frag = [&](int fs) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[fs][i], fb[fs][j], acc[i][j], 0, 0, 0);
  };
  // one K step on LDS buffer d & 1; ring slot (d + 1) % DEPTH holds the next tile.
  // MFMA fragments are double-buffered in registers: while the MFMAs of one 32-byte K
  // slice run, the LDS reads of the next slice, the LDS writes of the next tile and the
  // global loads of a later tile are issued in their shadow.  The first slice of a step
  // is read right after the barrier that publishes its tile.
  auto step_body = [&](int d) {
    const int buf = d & 1;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) read_frag(buf, kk + 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_frag(kk & 1);
      __builtin_amdgcn_sched_barrier(0);
      if (kk == 0) store_tile((d + 1) % DEPTH, buf ^ 1);
    }
    __syncthreads();
    read_frag(buf ^ 1, 0, 0);
  };

#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_tile(d, d);
  if (a.has_lut && tid < 64) lutw[tid] = lutv;   // (published by the first barrier of the K loop at the latest)
  if (PERSIST) {
    if (tid < BM) {
      qlds[tid] = qv[0];
      qlds[BM + tid] = qv[1];
      qlds[2 * BM + tid] = qv[2];
      qlds[3 * BM + tid] = qv[3];
    }
    __syncthreads();   // publishes qlds
  }

  // After the last barrier of a tile no wave reads LDS data it still needs, so the
  // first store of the next tile may overtake slower waves of the workgroup.
  for (;;) {
    // accumulators start from the bias (the int32 add of the epilogue commutes with the sum)
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const v4i *bp = PERSIST ? reinterpret_cast<const v4i *>(qlds + lch0 + i * 16)
                              : reinterpret_cast<const v4i *>(a.bias + ocw0 + i * 16);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i b = bp[q];
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          acc[i][j][q * 4 + 0] = b[0];
          acc[i][j][q * 4 + 1] = b[1];
          acc[i][j][q * 4 + 2] = b[2];
          acc[i][j][q * 4 + 3] = b[3];
        }
      }
    }
#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(1);
#endif
    store_tile(0, 0);
    __syncthreads();
#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(2);
#endif
    read_frag(0, 0, 0);

    // Whole groups of DEPTH steps: ring slots and LDS buffers are compile-time indices
    // (DEPTH is even, so buffer parity == slot parity) and the body has no branch.
    const int full = nsteps / DEPTH;
#pragma nounroll
    for (int g = 0; g < full; ++g) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        // slot d went to LDS one step ago: refill it with the tile DEPTH steps ahead
        load_tile(d, (g + 1) * DEPTH + d);
        step_body(d);
      }
    }
    // the last nsteps % DEPTH steps: their tiles are already in the ring / in LDS
    const int rem = nsteps - full * DEPTH;
#pragma unroll
    for (int d = 0; d < DEPTH - 1; ++d)
      if (d < rem) step_body(d);

#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(27);
#endif
    const int pix_done = pix0;
    bool more = false;
    if (PERSIST) {
      // next pixel tile of this workgroup: start its loads before the epilogue
      ltile += a.wgs_per_xcd;
      logical += a.wgs_per_xcd;
      more = ltile < a.tiles_per_xcd && logical < a.n_tiles;
      if (more) {
        pix0 += a.pstep_pix;
        ow_first += a.pstep_ow;
        if (ow_first >= a.ow) { ow_first -= a.ow; ++oh_first; }
        oh_first += a.pstep_oh;
        if (oh_first >= a.oh) { oh_first -= a.oh; ++n_first; }
        n_first += a.pstep_n;
        setup_rows();
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) load_tile(d, d);
      }
    }

    // the requantised tile goes through LDS (the K tiles' space: after the last barrier of the
    // K loop no wave needs them) and leaves in memory order
    int8_t *const stage = reinterpret_cast<int8_t *>(&lds[0][0]);
    static_assert(BN * stage_row_bytes<BM>() <= (int)sizeof(lds), "the staged tile must fit the K tiles");
    v4i sv[flush_chunks<BM, BN, NT>()];
    flush_prefetch<BM, BN, NT>(a, tid, pix_done, a.npix, oc0, out, sv);
    if (PERSIST)
      stage_rows<TM, TN, BM, FAST>(acc, a.relu_first, out.lo, stage, wn * TN * 32 + frow, lch0,
                                   qlds + BM + lch0, qlds + 2 * BM + lch0, qlds + 3 * BM + lch0);
    else
      stage_rows<TM, TN, BM, FAST>(acc, a.relu_first, out.lo, stage, wn * TN * 32 + frow, lch0,
                                   a.qmult + ocw0, a.qshift + ocw0, a.qhpot + ocw0);
#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(28);
#endif
    __syncthreads();
#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(29);
#endif
    flush_tile<BM, BN, NT>(a, stage, tid, pix_done, a.npix, oc0, out, lut, sv);
#ifdef TPUHIP_TRACE
    if (first_tile) TPUHIP_TS(30);
    first_tile = false;
    if (!PERSIST || !more) {
      ts[31] = (unsigned long long)clock64();
      if (a.trace && (tid & 63) == 0)
        for (int kq = 0; kq < 32; ++kq) a.trace[((size_t)blockIdx.x * 8 + (tid >> 6)) * 32 + kq] = ts[kq];
    }
#endif
    if (!PERSIST || !more) break;
    __syncthreads();   // the next tile's first K tile lands where the staged bytes are still read
  }
}

// ---------------------------------------------------------------------------
// 3x3 / stride 1 / pad 1 convolutions on feature maps narrow enough that a few whole
// rows fit a tile: the input patch of the tile ((TH + 2) rows x (W + 2) columns x C
// channels, borders zero) is fetched ONCE into LDS and the nine taps are formed from it,
// where the implicit-GEMM kernel above fetches every activation byte nine times.  Only
// the filter streams through the K loop (registers -> LDS, as above).  A workgroup
// computes BM output channels x TH rows of one image; pixels of the tile are its rows
// flattened, so they are consecutive in the output tensor too.
//   a.stem_pw = W + 2, a.magic_pw = floor(2^20 / (W + 2)) + 1, a.pstep_pix = TH,
//   a.pstep_n = tiles per image, a.pstep_oh = log2(C / 16), a.pstep_ow = swizzle shift
// C is 64, 128, 256 or 512 and a multiple of BK; the patch holds at most kPatchBytes (static
// LDS; with 256-byte K steps it is dynamic LDS of the layer's exact size, at most
// kPatchBytesDyn: a static array costs about half a microsecond less per launch).
// ---------------------------------------------------------------------------
constexpr int kPatchBytes = 45056;       // static patch (K steps up to 128 bytes)
constexpr int kPatchBytesDyn = 65536;    // dynamic patch (256-byte K steps: the filter tiles take 32 KB)

template <int BM, int BN, int BK, int DEPTH, int OCC, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void
conv_patch_kernel(ConvArgs a) {
  gather_conv_args(a);
  gather_conv_args_more(a);
  constexpr int WM = 2, WN = 2, NT = 256;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  constexpr int CH = BK / 16;
  constexpr int SW = CH == 4 ? 2 : CH == 8 ? 1 : 0;
  constexpr int RP = NT / CH;
  constexpr int NW = (BM + RP - 1) / RP;
  constexpr bool DYN = BK == 256;
  constexpr int NPL = (DYN ? kPatchBytesDyn : kPatchBytes) / 16 / NT;   // patch chunks per thread at most
  static_assert(TM >= 1 && TN >= 1, "bad tile");
  static_assert(DEPTH % 2 == 0 && DEPTH >= 2, "register ring depth");

  __shared__ v4i lds[2][BM * CH];
  __shared__ __attribute__((aligned(16))) int32_t qlds[4 * BM];
  __shared__ v4i patch_static[DYN ? 1 : kPatchBytes / 16];
  extern __shared__ __attribute__((aligned(16))) v4i patch_dynamic[];   // sized by the launch
  v4i *const patch = DYN ? patch_dynamic : patch_static;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int logical = (int)(blockIdx.x & 7) * a.tiles_per_xcd + (int)(blockIdx.x >> 3);
  if (logical >= a.n_tiles) return;
  const int pt = pixel_tile_of(a, logical);
  const int oc0 = (logical - pt * a.n_oc_tiles) * BM;
  const int img = pt / a.pstep_n;
  const int r0 = (pt - img * a.pstep_n) * a.pstep_pix;
  const int rows = min(a.pstep_pix, a.oh - r0);
  const int pix_base = (img * a.oh + r0) * a.ow;
  const int pix_limit = pix_base + rows * a.ow;
  const int pw = a.stem_pw;
  const int lg = a.pstep_oh, cht = 1 << lg, swp = a.pstep_ow;

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

  // ---- the patch: chunk q = position * (C / 16) + 16-channel group
  const int n_chunks = (a.pstep_pix + 2) * pw << lg;
  v4i preg[NPL];
#pragma unroll
  for (int u = 0; u < NPL; ++u) {
    const int q = tid + u * NT;
    const int pos = q >> lg, cc = q & (cht - 1);
    const int pr = (int)(((uint32_t)pos * a.magic_pw) >> 20);
    const int pc = pos - pr * pw;
    const int row = r0 - 1 + pr, col = pc - 1;
    const bool ok = q < n_chunks && (unsigned)row < (unsigned)a.ih && (unsigned)col < (unsigned)a.iw;
    preg[u] = buffer_load16(xrsrc, ok ? (uint32_t)(((img * a.ih + row) * a.iw + col) * a.x_cs + cc * 16)
                                      : kOobOffset);
  }

  int32_t qv[4] = {0, 0, 0, 0};
  static_assert(BM <= NT, "one parameter row per thread");
  if (tid < BM) {
    qv[0] = a.bias[oc0 + tid];
    qv[1] = a.qmult[oc0 + tid];
    qv[2] = a.qshift[oc0 + tid];
    qv[3] = a.qhpot[oc0 + tid];
  }

  // ---- the filter: as in conv_mfma_kernel
  const int kc = tid % CH;
  const int lrow = tid / CH;
  uint32_t woff[NW];
#pragma unroll
  for (int s = 0; s < NW; ++s) {
    const int r = lrow + RP * s;
    woff[s] = r < BM ? (uint32_t)((oc0 + r) * a.kp + kc * 16) : kOobOffset;
    asm volatile("" : "+v"(woff[s]));
  }
  v4i wreg[DEPTH][NW];
  const int nsteps = a.kp / BK;
  auto load_tile = [&](int slot, int step) {
    const bool in_k = step < nsteps;
#pragma unroll
    for (int s = 0; s < NW; ++s)
      wreg[slot][s] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
          wrsrc, in_k ? woff[s] : kOobOffset, step * BK, 0);
  };
  auto store_tile = [&](int slot, int buf) {
    v4i *base = lds[buf];
#pragma unroll
    for (int s = 0; s < NW; ++s) {
      const int r = lrow + RP * s;
      if (BM % RP == 0 || r < BM) base[r * CH + (kc ^ ((r >> SW) & (CH - 1)))] = wreg[slot][s];
    }
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_tile(d, d);

  const int frow = lane & 31;
  const int fk = lane >> 5;
  const int lch0 = wm * TM * 32 + fk * 16 * TM;
  const int ocw0 = oc0 + lch0;

  // top-left patch position of this lane's pixels (idle slots past the tile read position 0)
  int pos0[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int p = (wn * TN + j) * 32 + frow;
    const uint32_t pr = a.ow == 1 ? (uint32_t)p : __umulhi((uint32_t)p, a.magic_ow);
    const int pc = p - (int)pr * a.ow;
    pos0[j] = p < rows * a.ow ? (int)pr * pw + pc : 0;
  }

  // park the patch and the parameters
#pragma unroll
  for (int u = 0; u < NPL; ++u) {
    const int q = tid + u * NT;
    const int pos = q >> lg, cc = q & (cht - 1);
    if (q < n_chunks) patch[(pos << lg) + (cc ^ ((pos >> swp) & (cht - 1)))] = preg[u];
  }
  if (tid < BM) {
    qlds[tid] = qv[0];
    qlds[BM + tid] = qv[1];
    qlds[2 * BM + tid] = qv[2];
    qlds[3 * BM + tid] = qv[3];
  }

  v16i acc[TM][TN];
  constexpr int KK = BK / 32;
  v4i fa[2][TM], fb[2][TN];
  // fragments of 32-byte K slice kk of K step `step`: the filter from its LDS tile, the
  // activations from the patch at the step's tap
  auto read_frag = [&](int buf, int step, int kk, int fs) {
    const v4i *wl = lds[buf];
    const int chunk = kk * 2 + fk;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int r = (wm * TM + i) * 32 + frow;
      fa[fs][i] = wl[r * CH + (chunk ^ ((r >> SW) & (CH - 1)))];
    }
    const int kg0 = step * CH;
    const int tap = kg0 >> lg, cg = (kg0 & (cht - 1)) + chunk;
    const int tkh = (int)(((uint32_t)tap * a.magic_kw) >> 20);
    const int tap_off = tkh * pw + (tap - tkh * 3);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int pos = pos0[j] + tap_off;
      fb[fs][j] = patch[(pos << lg) + (cg ^ ((pos >> swp) & (cht - 1)))];
    }
  };
  auto mfma_frag = [&](int fs) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[fs][i], fb[fs][j], acc[i][j], 0, 0, 0);
  };
  int ks = 0;   // K step being multiplied
  auto step_body = [&](int d) {
    const int buf = d & 1;
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) read_frag(buf, ks, kk + 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
      mfma_frag(kk & 1);
      __builtin_amdgcn_sched_barrier(0);
      if (kk == 0) store_tile((d + 1) % DEPTH, buf ^ 1);
    }
    __syncthreads();
    ++ks;
    read_frag(buf ^ 1, min(ks, nsteps - 1), 0, 0);
  };

  __syncthreads();   // publishes qlds and the patch
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const v4i *bp = reinterpret_cast<const v4i *>(qlds + lch0 + i * 16);
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4i bq = bp[q];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j][q * 4 + 0] = bq[0];
        acc[i][j][q * 4 + 1] = bq[1];
        acc[i][j][q * 4 + 2] = bq[2];
        acc[i][j][q * 4 + 3] = bq[3];
      }
    }
  }
  store_tile(0, 0);
  __syncthreads();
  read_frag(0, 0, 0, 0);

  const int full = nsteps / DEPTH;
#pragma nounroll
  for (int g = 0; g < full; ++g) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      load_tile(d, (g + 1) * DEPTH + d);
      step_body(d);
    }
  }
  const int rem = nsteps - full * DEPTH;
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < rem) step_body(d);

  // the requantised tile goes through LDS (the patch's space: after the last barrier of the K
  // loop no wave needs it; the launch sizes a dynamic patch for the staged tile as well) and
  // leaves in memory order
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  int8_t *const stage = reinterpret_cast<int8_t *>(patch);
  static_assert(BN * stage_row_bytes<BM>() <= (DYN ? kPatchBytesDyn : kPatchBytes), "the staged tile must fit the patch");
  v4i sv[flush_chunks<BM, BN, NT>()];
  flush_prefetch<BM, BN, NT>(a, tid, pix_base, pix_limit, oc0, out, sv);
  stage_rows<TM, TN, BM, FAST>(acc, a.relu_first, out.lo, stage, wn * TN * 32 + frow, lch0, qlds + BM + lch0,
                               qlds + 2 * BM + lch0, qlds + 3 * BM + lch0);
  __syncthreads();
  flush_tile<BM, BN, NT>(a, stage, tid, pix_base, pix_limit, oc0, out, nullptr, sv);
}

// ---------------------------------------------------------------------------
// Pointwise (1x1, unpadded) convolutions with at most 256 input channels: the
// weights stay, the pixels stream.
//
// Most layers of a residual network are of this kind, and for them the multiply-adds are
// the small part: at K = 64 a 32x32 block of outputs costs two MFMAs (64 clocks) and about
// 500 clocks of requantisation on the vector ALU, and every byte of the big operand is
// used once.  So the kernel is laid out around the epilogue and the memory pipeline:
//   * a workgroup keeps its whole BM x K slice of the filter in LDS for its lifetime (the
//     image of that slice, swizzled, is what the packed filter holds: a straight copy) and
//     walks tiles of BN pixels; nothing of the filter is fetched per tile, no K loop with
//     barriers exists;
//   * the pixel rows of a tile are K contiguous bytes each, fetched with whole-row loads
//     (K / 16 neighbouring lanes per pixel) TWO tiles ahead into registers and parked in a
//     double-buffered LDS tile one tile ahead;
//   * the accumulators start at zero (the first MFMA of a block takes a literal 0) and the
//     bias rides in the 64-bit multiply-add of the requantisation: (acc + b) * m + 2^30 ==
//     acc * m + (b * m + 2^30), one per-channel 64-bit constant (needs the overflow-free
//     form of the layer, which the host proves; other layers take the general kernel);
//   * BM is as wide as the layer allows (up to 256 channels), so a tile's output -- and the
//     other operand of a fused add -- are whole rows of the tensors: staged through LDS,
//     read and written in memory order;
//   * one barrier per tile (the staged tile is double-buffered where LDS allows, SD == 2).
// K is padded to KP = 64, 128 or 256 with zero weights; the bytes a pixel row lacks are
// whatever follows it in memory (finite integers times zero; past the end of the tensor the
// buffer descriptor supplies zeros).
// ---------------------------------------------------------------------------
// Requantisation of accumulators that started at zero, for layers whose overflow-free form the
// host has proved: the bias rides in the addend of the 64-bit multiply-add,
//   (acc + b) * m + 2^30 == acc * m + c,   c = b * m + 2^30   (pc64: (low, high) pairs per channel).
// RELU (the layer clamps at 0 after saturation): the rounding right shift needs no sign term, as
// for x < 0 both (x + h) >> r and (x + h - 1) >> r are <= 0 and the clamp makes them 0; then
//   ((p >> 31) + h) >> r == (p + h * 2^31) >> (31 + r) == hi32(p + h * 2^31) >> (r - 1),   r >= 1,
// one multiply-add with c + h * 2^31 as the addend and one shift of the high word (pshift then
// holds r - 1 and phpot is not read).
// K slices by which the LDS reads of MFMA operands run ahead of their MFMAs: an LDS read takes
// some 130 clocks, a 32x32x32 MFMA 32 to 34
constexpr int frag_prefetch(int mfmas_per_slice) { return mfmas_per_slice >= 8 ? 1 : mfmas_per_slice >= 4 ? 2 : 3; }

template <int BM, int BN, int WM, int WN, int KP, int SD, int OCC>
__global__ __launch_bounds__(WM *WN * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void
conv_pw_kernel(ConvArgs a) {
  gather_conv_args(a);
  gather_conv_args_more(a);
  constexpr int NT = WM * WN * 64;
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert((WM * WN == 4 || WM * WN == 8) && TM >= 1 && TN >= 1 && TM * WM * 32 == BM && TN * WN * 32 == BN, "bad tile");
  static_assert(KP == 64 || KP == 128 || KP == 256, "padded K");
  static_assert(BM >= 64, "the threads that fetch the parameters also fetch the 64 table words");
  constexpr int KC = KP / 64;              // 64-byte K chunks
  constexpr int CPRK = KP / 16;            // 16-byte chunks of a pixel row
  constexpr int RPP = NT / CPRK;           // pixel rows per pass of the loader
  constexpr int NXC = (BN + RPP - 1) / RPP;   // activation chunks per thread per tile
  constexpr int WCH = BM * KP / 16;        // filter chunks of the slice
  constexpr int NWC = (WCH + NT - 1) / NT; // ... per thread
  constexpr bool XTAIL = BN % RPP != 0;    // the last pass covers fewer rows than threads
  constexpr int SROW = stage_row_bytes<BM>();
  extern __shared__ __attribute__((aligned(16))) v4i pw_smem[];
  v4i *const wA = pw_smem;                                       // [KC][BM][4 chunks], swizzled
  v4i *const xB = wA + KC * BM * 4;                              // [2][KC][BN][4 chunks], swizzled
  int8_t *const stage0 = reinterpret_cast<int8_t *>(xB + 2 * KC * BN * 4);   // [SD][BN][SROW]
  int32_t *const qlds = reinterpret_cast<int32_t *>(stage0 + SD * BN * SROW);   // 5 planes of BM
  uint32_t *const lutw = reinterpret_cast<uint32_t *>(qlds + 5 * BM);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  // tiles are dealt as in conv_mfma_kernel: every XCD a contiguous run of pixel tiles, a
  // workgroup keeps its output-channel tile and walks pixel tiles
  int ltile = (int)(blockIdx.x >> 3);
  int logical = (int)(blockIdx.x & 7) * a.tiles_per_xcd + ltile;
  if (logical >= a.n_tiles) return;
  const int pix_tile = pixel_tile_of(a, logical);
  const int oc0 = (logical - pix_tile * a.n_oc_tiles) * BM;
  const OutRoute out = route_out(a, __builtin_amdgcn_readfirstlane(oc0));
  int pix0 = pix_tile * BN;

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);

  // ---- loader: this thread fetches chunk c of pixel rows lrow + RPP * u
  const int c = tid % CPRK, lrow = tid / CPRK;
  int lpix0 = pix0;                       // first pixel of the tile being fetched
  // (stride 1: the input pixel has the output pixel's index, no coordinates at all -- three
  // divisions and the per-row arithmetic out of the path to the first load)
  int low = 0, loh = 0, ln = 0;
  if (!a.linear) {
    low = pix0 % a.ow;
    const int t = pix0 / a.ow;
    loh = t % a.oh;
    ln = t / a.oh;
  }
  v4i breg[NXC];
  auto load_B = [&](bool exists) {
#pragma unroll
    for (int u = 0; u < NXC; ++u) {
      const int row = lrow + RPP * u;
      const bool pv = exists && lpix0 + row < a.npix && (!XTAIL || row < BN);
      if (a.linear) {
        breg[u] = buffer_load16(xrsrc, pv ? (uint32_t)((lpix0 + row) * a.x_cs + c * 16) : kOobOffset);
        continue;
      }
      const uint32_t t1 = (uint32_t)(low + row);
      const uint32_t q1 = a.ow == 1 ? t1 : __umulhi(t1, a.magic_ow);
      const int ow = (int)(t1 - q1 * (uint32_t)a.ow);
      const uint32_t t2 = (uint32_t)loh + q1;
      const uint32_t q2 = a.oh == 1 ? t2 : __umulhi(t2, a.magic_oh);
      const int oh = (int)(t2 - q2 * (uint32_t)a.oh);
      const int n = ln + (int)q2;
      const uint32_t off = (uint32_t)(((n * a.ih + oh * a.sh) * a.iw + ow * a.sw) * a.x_cs + c * 16);
      breg[u] = buffer_load16(xrsrc, pv ? off : kOobOffset);
    }
  };
  auto advance_load = [&]() {
    lpix0 += a.pstep_pix;
    if (a.linear) return;
    low += a.pstep_ow;
    if (low >= a.ow) { low -= a.ow; ++loh; }
    loh += a.pstep_oh;
    if (loh >= a.oh) { loh -= a.oh; ++ln; }
    ln += a.pstep_n;
  };
  auto store_B = [&](int slot) {
    v4i *base = xB + slot * (KC * BN * 4) + (c >> 2) * (BN * 4);
#pragma unroll
    for (int u = 0; u < NXC; ++u) {
      const int row = lrow + RPP * u;
      if (!XTAIL || row < BN) base[row * 4 + ((c & 3) ^ ((row >> 2) & 3))] = breg[u];
    }
  };
  // does the tile j steps ahead of the current one exist?
  auto exists_ahead = [&](int j) {
    return ltile + j * a.wgs_per_xcd < a.tiles_per_xcd && logical + j * a.wgs_per_xcd < a.n_tiles;
  };

  load_B(true);
  {
    // the filter slice: a straight copy of its LDS image
    const v4i *wsrc = reinterpret_cast<const v4i *>(a.w) + (size_t)(oc0 / BM) * (BM * KP / 16);
    v4i wreg[NWC];
#pragma unroll
    for (int u = 0; u < NWC; ++u)
      if (WCH % NT == 0 || tid + u * NT < WCH) wreg[u] = wsrc[tid + u * NT];
    if (tid < BM) {
      // a workgroup whose result is clamped at 0 takes the constants of the short form
      const int32_t *c64 = out.lo == 0 ? a.qc64r : a.qc64;
      // all five in flight before the first is used (one trip to memory, not two)
      const int32_t c_lo = c64[2 * (oc0 + tid)], c_hi = c64[2 * (oc0 + tid) + 1];
      const int32_t qm = a.qmult[oc0 + tid], qs = a.qshift[oc0 + tid], qh = a.qhpot[oc0 + tid];
      uint32_t lutv = 0;
      if (a.has_lut && tid < 64) lutv = a.lut.w[tid];   // BM >= 64: these threads cover the table
      __builtin_amdgcn_sched_barrier(0);
      if (a.has_lut && tid < 64) lutw[tid] = lutv;
      qlds[2 * tid] = c_lo;
      qlds[2 * tid + 1] = c_hi;
      qlds[2 * BM + tid] = qm;
      qlds[3 * BM + tid] = qs - (out.lo == 0 ? 1 : 0);
      qlds[4 * BM + tid] = qh;
    }
#pragma unroll
    for (int u = 0; u < NWC; ++u)
      if (WCH % NT == 0 || tid + u * NT < WCH) wA[tid + u * NT] = wreg[u];
  }
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  store_B(0);
  advance_load();
  load_B(exists_ahead(1));
  __syncthreads();

  const int frow = lane & 31;
  const int fk = lane >> 5;
  const int lch0 = wm * TM * 32 + fk * 16 * TM;   // first of this lane's 16 * TM channels in the tile
  // fragment chunk indices (row * 4 + swizzled chunk) of this lane, for kk = 0 and 1
  int ia[TM][2], ib[TN][2];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int r = (wm * TM + i) * 32 + frow;
    ia[i][0] = r * 4 + (fk ^ ((r >> 2) & 3));
    ia[i][1] = r * 4 + ((2 + fk) ^ ((r >> 2) & 3));
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int r = (wn * TN + j) * 32 + frow;
    ib[j][0] = r * 4 + (fk ^ ((r >> 2) & 3));
    ib[j][1] = r * 4 + ((2 + fk) ^ ((r >> 2) & 3));
  }

  int cur = 0, sd = 0;
  for (;;) {
    v16i acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    const v4i *xb = xB + cur * (KC * BN * 4);
    // the operands of 32-byte K slice ks are requested PD slices before their MFMAs: with one
    // or two waves on a SIMD nothing else hides the LDS latency (two MFMAs take 64 clocks, an
    // LDS read twice that)
    constexpr int PD0 = OCC >= 4 ? 1 : frag_prefetch(TM * TN);
    constexpr int NS = KC * 2, PD = PD0 < NS ? PD0 : NS;
    v4i fa[PD + 1][TM], fb[PD + 1][TN];
    auto read_slice = [&](int ks, int slot) {
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[slot][i] = wA[(ks >> 1) * (BM * 4) + ia[i][ks & 1]];
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[slot][j] = xb[(ks >> 1) * (BN * 4) + ib[j][ks & 1]];
    };
#pragma unroll
    for (int ks = 0; ks < PD; ++ks) read_slice(ks, ks);
#pragma unroll
    for (int ks = 0; ks < NS; ++ks) {
      if (ks + PD < NS) read_slice(ks + PD, (ks + PD) % (PD + 1));
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[ks % (PD + 1)][i], fb[ks % (PD + 1)][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }

    // the next tile's pixels go to the other LDS tile (free since the barrier of the last
    // epilogue), the one after that is requested
    const bool more = exists_ahead(1);
    store_B(cur ^ 1);
    advance_load();
    load_B(exists_ahead(2));

    int8_t *const stage = stage0 + sd * (BN * SROW);
    v4i sv[flush_chunks<BM, BN, NT>()];
    flush_prefetch<BM, BN, NT>(a, tid, pix0, a.npix, oc0, out, sv);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      uint32_t outw[TN][4];
      const int lc = lch0 + i * 16;
      if (out.lo == 0)
        requant_rows_c64<TN, true>(acc[i], 0, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc,
                                   qlds + 4 * BM + lc, outw);
      else
        requant_rows_c64<TN, false>(acc[i], out.lo, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc,
                                    qlds + 4 * BM + lc, outw);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        *reinterpret_cast<v4i *>(stage + ((wn * TN + j) * 32 + frow) * SROW + lc) =
            v4i{(int)outw[j][0], (int)outw[j][1], (int)outw[j][2], (int)outw[j][3]};
    }
    __syncthreads();   // publishes the staged tile and the next tile's pixels
    flush_tile<BM, BN, NT>(a, stage, tid, pix0, a.npix, oc0, out, lut, sv);
    if (!more) break;
    ltile += a.wgs_per_xcd;
    logical += a.wgs_per_xcd;
    pix0 += a.pstep_pix;
    cur ^= 1;
    if (SD == 2) sd ^= 1;
    else __syncthreads();   // one staging area: everyone has read it before it is written again
  }
}

// ---------------------------------------------------------------------------
// 3x3 / stride 1 / pad 1 convolutions, second form of the row-patch kernel: the same tiling
// as conv_patch_kernel (a workgroup computes BM channels of TH whole rows of one image from a
// patch of TH + 2 input rows held in LDS, the filter streams through a double-buffered LDS
// tile), rebuilt around what the counters showed the first form spends its time on -- vector
// ALU instructions that are not arithmetic of the layer:
//   * LDS rows are PADDED by 16 bytes (patch position: C + 16 bytes, filter row: BK + 16)
//     instead of XOR-swizzled: 16 consecutive rows still start in 16 different 16-byte bank
//     groups (C and BK are multiples of 64), and an operand address becomes lane base +
//     wave-uniform offset -- one add per fragment and K step, immediates within a step --
//     where the swizzle cost five operations per fragment;
//   * the patch is fetched row by row: a lane's global offset is row base + 16 * index;
//   * K steps of BK = 128 or 256 bytes whatever the channel count (a step of a 64-channel
//     layer spans four taps), so a 3x3 x 64 layer meets three barriers, not nine;
//   * accumulators start at zero and the bias rides in the requantisation's 64-bit addend;
//     layers with a ReLU take the two-instruction form of requant_rows_c64.
// Layers whose overflow-free requantisation the host cannot prove stay with the first form.
//   a.stem_pw = W + 2, a.magic_pw = floor(2^20 / (W + 2)) + 1, a.pstep_pix = TH,
//   a.pstep_n = tiles per image, a.pstep_oh = log2(C), C a power of two from 64 to 1024
// LDS (dynamic): parameters | two filter tiles | patch; the staged output tile takes the
// filter tiles' place.
// ---------------------------------------------------------------------------
// 2 * (C + 16) + kPatch2RowPad is a multiple of 128 for every C that is a multiple of 64
constexpr int kPatch2RowPad = 96;

template <int BM, int BN, int WM, int WN, int BK, int OCC>
__global__ __launch_bounds__(WM *WN * 64) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void
conv_patch2_kernel(ConvArgs a) {
#ifdef TPUHIP_TRACE
  unsigned long long ts[32] = {};
#endif
  TPUHIP_TS(0);
  gather_conv_args(a);
  gather_conv_args_more(a);
  constexpr int NT = WM * WN * 64;
  constexpr int RD = 4;                       // filter tiles in flight in registers (even)
  constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert((WM * WN == 4 || WM * WN == 8) && TM >= 1 && TN >= 1 && TM * WM * 32 == BM && TN * WN * 32 == BN, "bad tile");
  static_assert(BK == 128 || BK == 256, "K bytes per step");
  constexpr int AROW = BK + 16;               // bytes of a filter tile row in LDS
  constexpr int ABYTES = BM * AROW;
  constexpr int CPA = BK / 16;                // 16-byte chunks of a filter tile row
  constexpr int NW = BM * CPA / NT;           // filter chunks per thread per step
  constexpr int KK = BK / 32;
  constexpr int NPL = 18 * 256 / NT;          // patch chunks per thread at most (72 KiB of input)
  static_assert(BN * stage_row_bytes<BM>() <= 2 * ABYTES, "the staged tile must fit the filter tiles");
  extern __shared__ __attribute__((aligned(16))) v4i p2_smem[];
  int32_t *const qlds = reinterpret_cast<int32_t *>(p2_smem);                 // 5 * BM dwords
  uint32_t *const lutw = reinterpret_cast<uint32_t *>(qlds + 5 * BM);         // 64 dwords
  int8_t *const abuf = reinterpret_cast<int8_t *>(lutw + 64);                 // 2 * ABYTES
  int8_t *const patch = abuf + 2 * ABYTES;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int logical = (int)(blockIdx.x & 7) * a.tiles_per_xcd + (int)(blockIdx.x >> 3);
  if (logical >= a.n_tiles) return;
  const int pt = pixel_tile_of(a, logical);
  const int oc0 = (logical - pt * a.n_oc_tiles) * BM;
  const int img = pt / a.pstep_n;
  const int r0 = (pt - img * a.pstep_n) * a.pstep_pix;
  const int rows = min(a.pstep_pix, a.oh - r0);
  const int pix_base = (img * a.oh + r0) * a.ow;
  const int pix_limit = pix_base + rows * a.ow;
  const int pw = a.stem_pw;
  const int lgc = a.pstep_oh;                 // log2(C)
  const int C = 1 << lgc;
  const int prow = C + 16;                    // bytes of a patch position in LDS
  // bytes of a patch row: its pw positions and kPatch2RowPad more, which make the pitch congruent to
  // ow positions modulo the 128 bytes of a bank sweep -- the 32 pixels of a fragment read, which wrap
  // from one image row into the next on narrow maps, then fall into banks as if they were consecutive
  // positions, wherever the wraps lie
  const int rowb = pw * prow + kPatch2RowPad;
  const bool relu = a.lo == 0;

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

  // the requantisation parameters and the fused table are requested first and parked last: loads
  // return in order, and nothing then waits for these alone
  int32_t qv[5] = {0, 0, 0, 0, 0};
  uint32_t lutv = 0;
  if (tid < BM) {
    const int32_t *c64 = relu ? a.qc64r : a.qc64;
    qv[0] = c64[2 * (oc0 + tid)];
    qv[1] = c64[2 * (oc0 + tid) + 1];
    qv[2] = a.qmult[oc0 + tid];
    qv[3] = a.qshift[oc0 + tid];
    qv[4] = a.qhpot[oc0 + tid];
  }
  if (a.has_lut && tid < 64) lutv = a.lut.w[tid];

  // ---- the patch: row r of it is pw positions of C bytes = pw * C / 16 chunks, of which chunk
  // p lies at byte (p - C / 16) * 16 of input row r0 - 1 + r (the first and last position are
  // the zero border)
  const int rowchunks = pw << (lgc - 4);
  const int n_chunks = (a.pstep_pix + 2) * rowchunks;
  v4i preg[NPL];
#pragma unroll
  for (int u = 0; u < NPL; ++u) {
    const int q = tid + u * NT;
    const int pr = (int)__umulhi((uint32_t)q, a.magic_c16);      // q / rowchunks
    const int p = q - pr * rowchunks;
    const int row = r0 - 1 + pr;
    const bool ok = q < n_chunks && (unsigned)row < (unsigned)a.ih && p >= (C >> 4) && p < ((a.iw + 1) << (lgc - 4));
    preg[u] = buffer_load16(xrsrc, ok ? (uint32_t)(((img * a.ih + row) * a.iw - 1) * C + p * 16) : kOobOffset);
  }

  // ---- the filter: K step s of this output-channel tile is BM * BK contiguous bytes
  static_assert(NW >= 1, "filter tile smaller than a pass of the workgroup");
  const uint32_t wbase = (uint32_t)(oc0 / BM) * (uint32_t)(a.kp * BM) + (uint32_t)tid * 16u;
  const int nsteps = a.kp / BK;
  v4i wr[RD][NW];
  // (no branch around a load: a step past the end of K reads zeros through the descriptor, so
  // that every step issues the same loads and the waits before the LDS stores count loads
  // instead of draining the queue.  The lane offsets are computed once and stay in their own
  // registers (an offset formed per load tends to land in the registers the load is about to
  // write, and the write-after-write wait that follows drains the queue just as well); a step
  // past the end takes an empty descriptor, a scalar select.)
  const __amdgpu_buffer_rsrc_t wnone = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, 0, 0x00020000);
  uint32_t woffs[NW];
#pragma unroll
  for (int u = 0; u < NW; ++u) {
    woffs[u] = wbase + (uint32_t)(u * NT * 16);
    asm volatile("" : "+v"(woffs[u]));
  }
  auto load_A = [&](int slot, int step) {
    const bool in_k = step < nsteps;
#pragma unroll
    for (int u = 0; u < NW; ++u)
      wr[slot][u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(in_k ? wrsrc : wnone, woffs[u], step * (BM * BK), 0);
  };
  auto store_A = [&](int slot, int buf) {
#pragma unroll
    for (int u = 0; u < NW; ++u) {
      const int q = tid + u * NT;
      *reinterpret_cast<v4i *>(abuf + buf * ABYTES + (q / CPA) * AROW + (q % CPA) * 16) = wr[slot][u];
    }
  };
#pragma unroll
  for (int d = 0; d < RD; ++d) load_A(d, d);

  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;

  const int frow = lane & 31;
  const int fk = lane >> 5;
  const int lch0 = wm * TM * 32 + fk * 16 * TM;
  // lane bases of the fragment reads
  int abase[TM], bbase[TN];
#pragma unroll
  for (int i = 0; i < TM; ++i) abase[i] = ((wm * TM + i) * 32 + frow) * AROW + fk * 16;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int p = (wn * TN + j) * 32 + frow;
    const uint32_t pr = a.ow == 1 ? (uint32_t)p : __umulhi((uint32_t)p, a.magic_ow);
    const int pc = p - (int)pr * a.ow;
    bbase[j] = (p < rows * a.ow ? (int)pr * rowb + pc * prow : 0) + fk * 16;   // idle slots read position 0
  }

  // park the patch and the first filter tile
#pragma unroll
  for (int u = 0; u < NPL; ++u) {
    const int q = tid + u * NT;
    const int pr = (int)__umulhi((uint32_t)q, a.magic_c16);
    const int p = q - pr * rowchunks;
    if (q < n_chunks)
      *reinterpret_cast<v4i *>(patch + pr * rowb + (p >> (lgc - 4)) * prow + (p & ((C >> 4) - 1)) * 16) = preg[u];
  }
  if (tid < BM) {
    qlds[2 * tid] = qv[0];
    qlds[2 * tid + 1] = qv[1];
    qlds[2 * BM + tid] = qv[2];
    qlds[3 * BM + tid] = qv[3] - (relu ? 1 : 0);
    qlds[4 * BM + tid] = qv[4];
  }
  if (a.has_lut && tid < 64) lutw[tid] = lutv;
  TPUHIP_TS(1);
  store_A(0, 0);
  __syncthreads();
  TPUHIP_TS(2);

  // A wave whose tile is a single 32x32 block would issue its MFMAs as one dependent chain (every
  // MFMA waits for the one before); it keeps two sets of accumulators and alternates between them
  // by K slice -- two independent chains -- and adds them up before the requantisation.
  constexpr int NACC = TM * TN == 1 ? 2 : 1;
  v16i accs[NACC][TM][TN];
#pragma unroll
  for (int c = 0; c < NACC; ++c)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) accs[c][i][j][e] = 0;
  v16i (&acc)[TM][TN] = accs[0];

  // One K step; its register slot (compile-time, step % RD) is free -- its tile went to LDS a
  // step ago -- and receives the tile RD steps ahead; the next step's tile goes from its slot
  // to the other LDS tile.  Within the step the operands of a 32-byte K slice are requested PD
  // slices before their MFMAs (see frag_prefetch).
  constexpr int PD = OCC >= 4 ? 1 : frag_prefetch(TM * TN);
  auto step = [&](int s, auto slotc) {
    constexpr int slot = decltype(slotc)::value, buf = slot & 1;
#ifdef TPUHIP_TRACE
    const bool tr = s < 4;
    if (tr) TPUHIP_TS(3 + slot * 6);
#endif
    load_A(slot, s + RD);
    const int8_t *ab = abuf + buf * ABYTES;
    v4i fa[PD + 1][TM], fb[PD + 1][TN];
    auto read_slice = [&](int kk, int fs) {
      // the slice lies in one filter tap (C is a multiple of 64); slices past the ninth tap
      // meet zero weights and read the last tap
      const int koff = s * BK + kk * 32;
      const int tap = min(koff >> lgc, 8);
      const int tkh = (tap * 11) >> 5;
      const int boff = tkh * rowb + (tap - 3 * tkh) * prow + (koff & (C - 1));
#pragma unroll
      for (int i = 0; i < TM; ++i) fa[fs][i] = *reinterpret_cast<const v4i *>(ab + abase[i] + kk * 32);
#pragma unroll
      for (int j = 0; j < TN; ++j) fb[fs][j] = *reinterpret_cast<const v4i *>(patch + bbase[j] + boff);
    };
    // K is padded to whole steps with zero weights: the slices of the last step that lie in
    // the padding are not multiplied (kreal: slices of this step that hold weights)
    const int kreal = min(KK, (a.k16 * 16 - s * BK + 31) >> 5);
#pragma unroll
    for (int kk = 0; kk < PD; ++kk) read_slice(kk, kk);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + PD < KK) read_slice(kk + PD, (kk + PD) % (PD + 1));
      __builtin_amdgcn_sched_barrier(0);
      if (kk < kreal) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            accs[kk % NACC][i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[kk % (PD + 1)][i], fb[kk % (PD + 1)][j],
                                                                          accs[kk % NACC][i][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
#ifdef TPUHIP_TRACE
      if (tr && kk == 0) TPUHIP_TS(4 + slot * 6);
      if (tr && kk == 3) TPUHIP_TS(5 + slot * 6);
      if (tr && kk == KK - 1) TPUHIP_TS(6 + slot * 6);
#endif
    }
    store_A((slot + 1) % RD, buf ^ 1);   // (past the last step: zeros, into a tile nobody reads)
#ifdef TPUHIP_TRACE
    if (tr) TPUHIP_TS(7 + slot * 6);
#endif
    __syncthreads();
#ifdef TPUHIP_TRACE
    if (tr) TPUHIP_TS(8 + slot * 6);
#endif
  };
  for (int s = 0; s < nsteps; s += RD) {
    step(s, std::integral_constant<int, 0>{});
    if (s + 1 < nsteps) step(s + 1, std::integral_constant<int, 1>{});
    if (s + 2 < nsteps) step(s + 2, std::integral_constant<int, 2>{});
    if (s + 3 < nsteps) step(s + 3, std::integral_constant<int, 3>{});
  }

  TPUHIP_TS(27);
  if (NACC == 2) {
#pragma unroll
    for (int e = 0; e < 16; ++e) accs[0][0][0][e] += accs[NACC - 1][0][0][e];
  }
  // the requantised tile goes through LDS (the filter tiles' space: every wave is past the
  // last barrier of the K loop) and leaves in memory order
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  int8_t *const stage = abuf;
  v4i sv[flush_chunks<BM, BN, NT>()];
  flush_prefetch<BM, BN, NT>(a, tid, pix_base, pix_limit, oc0, out, sv);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    uint32_t outw[TN][4];
    const int lc = lch0 + i * 16;
    if (relu)
      requant_rows_c64<TN, true>(acc[i], 0, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc, qlds + 4 * BM + lc, outw);
    else
      requant_rows_c64<TN, false>(acc[i], a.lo, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc, qlds + 4 * BM + lc,
                                  outw);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      *reinterpret_cast<v4i *>(stage + ((wn * TN + j) * 32 + frow) * stage_row_bytes<BM>() + lc) =
          v4i{(int)outw[j][0], (int)outw[j][1], (int)outw[j][2], (int)outw[j][3]};
  }
  TPUHIP_TS(28);
  __syncthreads();
  TPUHIP_TS(29);
  flush_tile<BM, BN, NT>(a, stage, tid, pix_base, pix_limit, oc0, out, lut, sv);
  TPUHIP_TS(30);
#ifdef TPUHIP_TRACE
  if (a.trace && (tid & 63) == 0) {
    for (int k = 0; k < 32; ++k) a.trace[((size_t)blockIdx.x * 8 + (tid >> 6)) * 32 + k] = ts[k];
  }
#endif
}

// ---------------------------------------------------------------------------
// 3x3 / stride 1 / pad 1 convolutions, third form of the row-patch kernel, for layers whose K is
// long and whose pixels are few (the late stages of a residual network, 14x14 and 7x7 maps):
// there the second form spends its time between barriers -- nine and more K steps, each a
// filter tile parked in LDS, a barrier, and an LDS round trip before the first MFMA -- and on
// LDS reads, two fragments per MFMA.  Here the K loop has no barrier and no filter in LDS:
//   * a workgroup of four waves computes 32 output channels of a tile of whole rows of one image
//     (or of a few whole images, where two and more fit the tile's NBLK x 32 pixel slots) from
//     the input patch held in LDS, laid out as in the second form;
//   * the four waves SPLIT K: wave w multiplies 32-byte K slices w, w + 4, w + 8, ... for ALL
//     pixel blocks of the tile.  Its filter operand of a slice is one MFMA A fragment, which the
//     packed filter holds as 1 KB contiguous in memory ([channel block][slice][lane][16 bytes]):
//     one coalesced load per slice straight into registers, U slices ahead, read by this wave
//     alone.  One A fragment then meets NBLK B fragments from the patch: NBLK MFMAs per
//     NBLK + 1 operand reads, and independent accumulators back to back;
//   * the partial sums meet in LDS (the patch's space): every wave parks the blocks it does not
//     own, a barrier, and the owner of a block (wave j & 3 for block j) adds the three others';
//   * requantisation and the staged, row-ordered output as in the other LDS kernels (fused
//     table and add included).
// OB = 2: the workgroup computes 64 channels, every wave two A fragments per slice against the
// same NBLK B fragments (2 * NBLK MFMAs per NBLK + 2 operand reads).  A workgroup then fetches
// its patch once for twice the channels: on maps whose patch is large against the filter slice
// (19x19 x 512 channels: 134 KB per tile) the launch is bound by what the CUs can pull out of
// L2, patches and filter fragments together, and this form moves about half of it.  The partial
// sums meet in one round per channel block (the space holds one block's guests).
//   a.stem_pw = W + 2, a.pstep_pix = TH (rows of a tile), a.pstep_n = tiles per image,
//   a.tile_imgs = whole images per tile (1: a tile is TH rows of one image),
//   a.pstep_oh = log2(C), a.magic_c16 = ceil(2^32 / 16-byte chunks of an input row),
//   a.magic_kw = ceil(2^32 / H), a.magic_oh = ceil(2^32 / (H * W)), a.pstep_ow = LDS bytes
// LDS (dynamic): parameters | table | patch, then the partial sums, then the staged tile.
// ---------------------------------------------------------------------------
template <int NB2, int PW, int OB>
__global__ __launch_bounds__(256 * PW) void conv_patch3_kernel(ConvArgs a) {
#ifdef TPUHIP_TRACE
  unsigned long long ts[32] = {};
#endif
  TPUHIP_TS(0);
  gather_conv_args(a);
  gather_conv_args_more(a);
  // 4 * PW waves: wave = pixel group * 4 + K group; a pixel group is NB2 blocks of 32 pixel slots
  constexpr int NT = 256 * PW, NWAVES = 4 * PW, BM = 32 * OB, BN = NB2 * PW * 32;
  constexpr int U = OB == 1 ? 8 : 4;   // K slices in flight per wave (even), OB A fragments each
  constexpr int NPL = 16 / PW;  // pieces of the input span per wave and pass
  extern __shared__ __attribute__((aligned(16))) v4i p3_smem[];
  int32_t *const qlds = reinterpret_cast<int32_t *>(p3_smem);                 // 5 * BM dwords
  uint32_t *const lutw = reinterpret_cast<uint32_t *>(qlds + 5 * BM);         // 64 dwords
  int8_t *const patch = reinterpret_cast<int8_t *>(lutw + 64);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kg = wave & 3;          // K group: slices kg, kg + 4, ...
  const int pg = wave >> 2;         // pixel group: blocks pg * NB2 ...
  const int logical = (int)(blockIdx.x & 7) * a.tiles_per_xcd + (int)(blockIdx.x >> 3);
  if (logical >= a.n_tiles) return;
  const int pt = pixel_tile_of(a, logical);
  const int ocb = logical - pt * a.n_oc_tiles;
  const int oc0 = ocb * BM;
  const int imgs = a.tile_imgs;
  int img0, r0, rows, nimg;
  if (imgs > 1) {
    img0 = pt * imgs; r0 = 0; rows = a.oh; nimg = min(imgs, a.n - img0);
  } else {
    img0 = pt / a.pstep_n; r0 = (pt - img0 * a.pstep_n) * a.pstep_pix; rows = min(a.pstep_pix, a.oh - r0); nimg = 1;
  }
  const int pix_base = (img0 * a.oh + r0) * a.ow;
  const int npx = nimg * rows * a.ow;
  const int pix_limit = pix_base + npx;
  const int pw = a.stem_pw;
  const int lgc = a.pstep_oh;                 // log2(C)
  const int C = 1 << lgc;
  const int prow = C + 16;                    // bytes of a patch position in LDS
  const int rowb = pw * prow + kPatch2RowPad; // bytes of a patch row (see conv_patch2_kernel)
  const int th2 = a.pstep_pix + 2;            // patch rows per image
  const bool relu = a.lo == 0;
  // blocks of this wave's pixel group that hold pixels
  const int nb = min(NB2, ((npx + 31) >> 5) - pg * NB2);

  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wnone = __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, 0, 0x00020000);

  // the requantisation parameters are requested first and parked last: loads return in order,
  // and nothing then waits for these alone
  int32_t qv[5] = {0, 0, 0, 0, 0};
  if (tid < BM) {
    const int32_t *c64 = relu ? a.qc64r : a.qc64;
    qv[0] = c64[2 * (oc0 + tid)];
    qv[1] = c64[2 * (oc0 + tid) + 1];
    qv[2] = a.qmult[oc0 + tid];
    qv[3] = a.qshift[oc0 + tid];
    qv[4] = a.qhpot[oc0 + tid];
  }
  uint32_t lutv = 0;
  if (a.has_lut && tid < 64) lutv = a.lut.w[tid];

  // ---- the filter: slice sl of this channel block is the 1 KB fragment (ocb * nsl + sl)
  const int nsl = a.kp >> 5;
  const int trips = nb > 0 ? (nsl - kg + 3) >> 2 : 0;   // slices kg, kg + 4, ... below nsl
  uint32_t wlane = (uint32_t)lane * 16u;
  asm volatile("" : "+v"(wlane));
  const uint32_t wblock = (uint32_t)(ocb * OB) * (uint32_t)nsl * 1024u;   // block ob of the tile: nsl KB further each
  // (a request past the wave's last slice repeats the last one: same loads every trip, never used)
  auto load_A = [&](v4i (&dst)[OB], int i) {
    const int sl = kg + 4 * min(i, trips - 1);
#pragma unroll
    for (int ob = 0; ob < OB; ++ob)
      dst[ob] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(trips > 0 ? wrsrc : wnone, wlane,
                                                           wblock + (uint32_t)(ob * nsl + sl) * 1024u, 0);
  };
  v4i af[U][OB];
#pragma unroll
  for (int u = 0; u < U; ++u) load_A(af[u], u);

  // ---- the patch.  Patch row pr (image pr / th2 of the tile, input row r0 - 1 + pr % th2) is pw
  // positions of C bytes; positions 1 .. W are the input row (W * C contiguous bytes), the
  // first and last position and the rows outside the image are the zero border.  The input rows
  // a tile needs are ONE contiguous span of x (consecutive rows of an image, consecutive whole
  // images), so the span is fetched as a byte stream: wave w takes its 1 KB pieces w, w + NWAVES,
  // ... through a descriptor that begins at the piece and ends with the span (a piece past the
  // end: nothing), every lane 16 bytes at one fixed offset -- scalar work and no branch per
  // load -- and each lane finds the patch position of its chunk (row = chunk / chunks of a row)
  // when it parks it.  NPL pieces per wave are in flight at a time.  The whole patch is zeroed
  // first (border positions, rows outside the image, images the last tile lacks).
  TPUHIP_TS(13);
  {
    const int cshift = lgc - 4;
    const int chunks_in = a.iw << cshift;                 // chunks of an input row
    // first and last input row of the span (single image), or all rows of the tile's images
    const int row_f = imgs > 1 ? 0 : max(r0 - 1, 0);
    const int row_l = imgs > 1 ? nimg * a.ih - 1 : min(r0 + rows, a.ih - 1);
    const int span_chunks = (row_l - row_f + 1) * chunks_in;
    const int span_bytes = span_chunks << 4;
    const int8_t *span = a.x + ((size_t)((img0 * a.ih + row_f) * a.iw) << lgc);
    const int pieces = (span_bytes + 1023) >> 10;
    uint32_t lane16 = (uint32_t)lane * 16u;
    asm volatile("" : "+v"(lane16));
    const int total_chunks = imgs * th2 * rowb >> 4;      // (rowb is a multiple of 16)
    // (every wave makes the first pass, whatever the span: the barrier inside is the workgroup's)
    int piece0 = wave;
    do {
      v4i preg[NPL];
#pragma unroll
      for (int u = 0; u < NPL; ++u) {
        const int off = (piece0 + u * NWAVES) << 10;
        const __amdgpu_buffer_rsrc_t rs =
            __builtin_amdgcn_make_buffer_rsrc((void *)(span + min(off, span_bytes)), 0, max(span_bytes - off, 0), 0x00020000);
        preg[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(rs, lane16, 0, 0);
      }
      if (piece0 == wave) {
        // (first pass only) the zeros, and the barrier that orders them before the data
        for (int q = tid; q < total_chunks; q += NT) *reinterpret_cast<v4i *>(patch + q * 16) = v4i{0, 0, 0, 0};
        __syncthreads();
      }
#ifdef TPUHIP_TRACE
      if (piece0 == wave) TPUHIP_TS(14);
#endif
#pragma unroll
      for (int u = 0; u < NPL; ++u) {
        const int c = ((piece0 + u * NWAVES) << 6) + lane;                 // chunk of the span
        const int g = (int)__umulhi((uint32_t)c, a.magic_c16);            // its row in the span
        const int p = c - g * chunks_in;
        // patch row: a single image's span begins at patch row row_f - (r0 - 1); whole images
        // have a border row before and after each
        // (x / d by umulhi(x, ceil(2^32 / d)) has no constant for d == 1)
        const int pr = imgs > 1 ? g + 1 + 2 * (a.ih == 1 ? g : (int)__umulhi((uint32_t)g, a.magic_kw)) : g + row_f - (r0 - 1);
        if (c < span_chunks)
          *reinterpret_cast<v4i *>(patch + pr * rowb + prow + p * 16 + ((p >> cshift) << 4)) = preg[u];
#ifdef TPUHIP_TRACE
        if (piece0 == wave && u == 0) TPUHIP_TS(15);
        if (piece0 == wave && u == 7) TPUHIP_TS(16);
#endif
      }
      piece0 += NWAVES * NPL;
    } while (piece0 < pieces);
  }

  if (tid < BM) {
    qlds[2 * tid] = qv[0];
    qlds[2 * tid + 1] = qv[1];
    qlds[2 * BM + tid] = qv[2];
    qlds[3 * BM + tid] = qv[3] - (relu ? 1 : 0);
    qlds[4 * BM + tid] = qv[4];
  }
  if (a.has_lut && tid < 64) lutw[tid] = lutv;
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;

  const int frow = lane & 31;
  const int fk = lane >> 5;
  // lane bases of the B fragment reads: pixel slot p of the tile -> its patch position
  int bbase[NB2];
  const int ohow = a.oh * a.ow;
#pragma unroll
  for (int j = 0; j < NB2; ++j) {
    const int p = (pg * NB2 + j) * 32 + frow;
    const int il = imgs > 1 ? (ohow == 1 ? p : (int)__umulhi((uint32_t)p, a.magic_oh)) : 0;   // p / (H * W)
    const int rem = p - il * ohow;
    const uint32_t pr = a.ow == 1 ? (uint32_t)rem : __umulhi((uint32_t)rem, a.magic_ow);
    const int pc = rem - (int)pr * a.ow;
    bbase[j] = (p < npx ? (il * th2 + (int)pr) * rowb + pc * prow : 0) + fk * 16;   // idle slots read position 0
  }
  TPUHIP_TS(1);
  __syncthreads();   // the patch and the parameters are in place
  TPUHIP_TS(2);

  v16i acc[OB][NB2];
#pragma unroll
  for (int ob = 0; ob < OB; ++ob)
#pragma unroll
    for (int j = 0; j < NB2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[ob][j][e] = 0;

  // The wave's slices advance by 128 bytes of K: the channel offset c0 within the tap and the
  // tap's patch offset are kept as scalars (taps past the ninth -- one read ahead of the last
  // slice -- stay on the ninth)
  int c0 = (kg * 32) & (C - 1), tap = (kg * 32) >> lgc;
  int tw = tap - 3 * ((tap * 11) >> 5);
  int tapoff = ((tap * 11) >> 5) * rowb + tw * prow;
  v4i bf[2][NB2];
  auto read_B = [&](int fs) {
    const int boff = tapoff + c0;
#pragma unroll
    for (int j = 0; j < NB2; ++j) bf[fs][j] = *reinterpret_cast<const v4i *>(patch + bbase[j] + boff);
    c0 += 128;
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      if (c0 >= C) {
        c0 -= C;
        if (tap < 8) {
          ++tap;
          if (++tw == 3) { tw = 0; tapoff += rowb - 2 * prow; } else tapoff += prow;
        }
      }
    }
  };
  if (trips > 0) read_B(0);
  // Whole rounds of U trips run without a branch inside: every trip consumes the fragment
  // requested U trips earlier and requests one, so the wait before a trip counts loads instead
  // of draining the queue.  The last trips (fewer than U) take what is already in registers.
  int i0 = 0;
  for (; i0 + U <= trips; i0 += U) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
#ifdef TPUHIP_TRACE
      if (i0 == 0) ts[3 + u] = (unsigned long long)clock64();
#endif
      read_B((u + 1) & 1);
      v4i afr[OB];
#pragma unroll
      for (int ob = 0; ob < OB; ++ob) afr[ob] = af[u][ob];
      load_A(af[u], i0 + u + U);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j = 0; j < NB2; ++j)
#pragma unroll
        for (int ob = 0; ob < OB; ++ob)
          acc[ob][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afr[ob], bf[u & 1][j], acc[ob][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#pragma unroll
  for (int u = 0; u < U - 1; ++u) {
    if (i0 + u >= trips) break;
    read_B((u + 1) & 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < NB2; ++j)
#pragma unroll
      for (int ob = 0; ob < OB; ++ob)
        acc[ob][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[u][ob], bf[u & 1][j], acc[ob][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }

  TPUHIP_TS(27);
  // ---- the four partial sums of every block meet at the block's owner, K group j & 3
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  v4i sv[flush_chunks<BM, BN, NT>()];
  flush_prefetch<BM, BN, NT>(a, tid, pix_base, pix_limit, oc0, out, sv);
  __syncthreads();   // every wave is done with the patch
  v4i *const red = reinterpret_cast<v4i *>(patch) + pg * (NB2 * 3 * 4 * 64);   // [block][3 guests][4 quads][64 lanes]
  // (one round per channel block of the wave: the space holds the guests' sums of NB2 blocks)
#pragma unroll
  for (int ob = 0; ob < OB; ++ob) {
#pragma unroll
    for (int j = 0; j < NB2; ++j) {
      if ((j & 3) != kg && j < nb) {
        const int slot = (kg - (j & 3) - 1) & 3;
#pragma unroll
        for (int q = 0; q < 4; ++q)
          red[((j * 3 + slot) * 4 + q) * 64 + lane] =
              v4i{acc[ob][j][q * 4], acc[ob][j][q * 4 + 1], acc[ob][j][q * 4 + 2], acc[ob][j][q * 4 + 3]};
      }
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < NB2; ++j) {
      if ((j & 3) == kg && j < nb) {
#pragma unroll
        for (int slot = 0; slot < 3; ++slot)
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const v4i v = red[((j * 3 + slot) * 4 + q) * 64 + lane];
            acc[ob][j][q * 4] += v[0]; acc[ob][j][q * 4 + 1] += v[1]; acc[ob][j][q * 4 + 2] += v[2]; acc[ob][j][q * 4 + 3] += v[3];
          }
      }
    }
    __syncthreads();   // the partial sums are read: their space takes the next round's, then the staged tile
  }
  TPUHIP_TS(28);

  // ---- requantisation into the staging area, then out in memory order (a lane's 16 results of
  // channel block ob are channels fk * 16 * OB + ob * 16 ... of the tile: see mfma_row_to_oc)
  int8_t *const stage = patch;
#pragma unroll
  for (int ob = 0; ob < OB; ++ob) {
    const int lc = fk * 16 * OB + ob * 16;
#pragma unroll
    for (int j = 0; j < NB2; ++j) {
      if ((j & 3) == kg && j < nb) {
        const v16i one[1] = {acc[ob][j]};
        uint32_t outw[1][4];
        if (relu)
          requant_rows_c64<1, true>(one, 0, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc, qlds + 4 * BM + lc, outw);
        else
          requant_rows_c64<1, false>(one, a.lo, qlds + 2 * lc, qlds + 2 * BM + lc, qlds + 3 * BM + lc, qlds + 4 * BM + lc, outw);
        *reinterpret_cast<v4i *>(stage + ((pg * NB2 + j) * 32 + frow) * stage_row_bytes<BM>() + lc) =
            v4i{(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
      }
    }
  }
  __syncthreads();
  TPUHIP_TS(29);
  flush_tile<BM, BN, NT>(a, stage, tid, pix_base, pix_limit, oc0, out, lut, sv);
  TPUHIP_TS(30);
#ifdef TPUHIP_TRACE
  if (a.trace && (tid & 63) == 0) {
    for (int k = 0; k < 32; ++k) a.trace[((size_t)blockIdx.x * 8 + (tid >> 6)) * 32 + k] = ts[k];
  }
#endif
}

// ---------------------------------------------------------------------------
// depthwise on the matrix cores.  A depthwise tap is a 32x32 DIAGONAL matrix times
// the 32 channels x 32 pixels activation block: D[c][pix] += W_t[c][c] * X_t[pix][c],
// one v_mfma_i32_32x32x32_i8 per tap (K = the 32 channels).  31/32 of the multiplies
// hit zeros, but the matrix pipe is otherwise idle here and the vector ALU, which the
// per-byte multiply-adds of the scalar form saturate, is left with the requantisation
// alone.  The B fragment of a tap is exactly a channels-last load (lane: pixel l & 31,
// 16 channels from 16*(l >> 5)); the diagonal A fragments are built on the host, rows
// permuted so that a lane's 16 results are 16 consecutive channels.  A wave keeps its
// 32-channel block and walks 32-pixel blocks.
// REGW: kh*kw <= 9 and the nine A fragments stay in registers.
// ---------------------------------------------------------------------------
template <bool FAST, bool REGW>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(REGW ? 3 : 4, REGW ? 3 : 4))) void
conv_depthwise_mfma_kernel(ConvArgs a) {
  __shared__ uint32_t lutw[64];
  __shared__ int32_t qlds[4][4][32];                  // per wave: bias, mult, shift, hpot
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int frow = lane & 31, fk = lane >> 5;
  const int n_cb = (a.ocw + 31) >> 5;
  // workgroups are dealt to the 8 XCDs round-robin; each XCD takes a contiguous run of pixel
  // blocks, so the input rows that vertically neighbouring blocks share meet in one L2
  const int n_pb_all = (a.npix + 31) >> 5;
  const int pb_per_xcd = (n_pb_all + 7) >> 3;
  const int xcd = (int)(blockIdx.x & 7);
  const int n_pb = min(n_pb_all, (xcd + 1) * pb_per_xcd);   // end of this XCD's run
  const int gw = (int)(blockIdx.x >> 3) * 4 + wave;          // wave index within the XCD
  const int nslots = (int)(gridDim.x >> 3) * 4 / n_cb;       // pixel blocks in flight per XCD (>= 1)
  const int cb = gw % n_cb;
  int pb = gw / n_cb;
  // a wave's parameters never change: they live in LDS, whose reads do not queue behind
  // the activation loads in flight (the parameter arrays are padded past the last block)
  {
    const int32_t *src = fk == 0 ? a.bias : a.qmult;
    const int32_t *src2 = fk == 0 ? a.qshift : a.qhpot;
    qlds[wave][fk][frow] = src[cb * 32 + frow];
    qlds[wave][2 + fk][frow] = src2[cb * 32 + frow];
  }
  if (a.has_lut && threadIdx.x < 64) lutw[threadIdx.x] = a.lut.w[threadIdx.x];
  __syncthreads();
  if (pb >= nslots) return;                           // no barrier below
  pb += xcd * pb_per_xcd;
  if (pb >= n_pb) return;
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  const int oc = cb * 32 + fk * 16;                   // this lane's 16 channels
  const bool ch_ok = oc < a.ocw;
  const int taps = a.kh * a.kw;
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const v4i *afrag = reinterpret_cast<const v4i *>(a.w) + (size_t)cb * taps * 64 + lane;
  v4i areg[REGW ? 9 : 1];
  if (REGW) {
#pragma unroll
    for (int t = 0; t < 9; ++t) areg[t] = t < taps ? afrag[t * 64] : v4i{0, 0, 0, 0};
  }
  const int32_t *pbias = &qlds[wave][0][fk * 16], *pmult = &qlds[wave][1][fk * 16];
  const int32_t *pshift = &qlds[wave][2][fk * 16], *phpot = &qlds[wave][3][fk * 16];

  int pix = pb * 32 + frow;
  int ow = pix % a.ow;
  int oh = (pix / a.ow) % a.oh;
  int n = pix / (a.ow * a.oh);
  const int step = nslots * 32;
  const int d_ow = step % a.ow, d_oh = (step / a.ow) % a.oh, d_n = step / (a.ow * a.oh);

  auto tap_load = [&](int t) {
    const int tkh = (int)(((uint32_t)t * a.magic_kw) >> 20);
    const int tkw = t - tkh * a.kw;
    const int ihb = oh * a.sh - a.pt, iwb = ow * a.sw - a.pl;
    const int ih = ihb + tkh * a.dh, iw = iwb + tkw * a.dw;
    const bool ok = (pix < a.npix) & ch_ok & (t < taps) & ((unsigned)ih < (unsigned)a.ih) &
                    ((unsigned)iw < (unsigned)a.iw);
    return buffer_load16(xrsrc, ok ? (uint32_t)(((n * a.ih + ih) * a.iw + iw) * a.x_cs + oc)
                                   : kOobOffset);
  };
  auto advance = [&]() {
    pb += nslots;
    pix += step;
    ow += d_ow;
    if (ow >= a.ow) { ow -= a.ow; ++oh; }
    oh += d_oh;
    if (oh >= a.oh) { oh -= a.oh; ++n; }
    n += d_n;
  };
  auto bias_acc = [&](v16i &acc) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4i b = *reinterpret_cast<const v4i *>(pbias + q * 4);
      acc[q * 4 + 0] = b[0]; acc[q * 4 + 1] = b[1]; acc[q * 4 + 2] = b[2]; acc[q * 4 + 3] = b[3];
    }
  };

  if (REGW) {
    // the nine operands of the NEXT pixel block are requested before the epilogue of this
    // one, into the registers the MFMAs have just consumed
    v4i bt[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) bt[t] = tap_load(t);
    for (;;) {
      v16i acc[1];
      bias_acc(acc[0]);
#pragma unroll
      for (int t = 0; t < 9; ++t)
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[t], bt[t], acc[0], 0, 0, 0);
      const int pix_done = pix;
      advance();
      const bool more = pb < n_pb;
      if (more) {
#pragma unroll
        for (int t = 0; t < 9; ++t) bt[t] = tap_load(t);
      }
      if (ch_ok) epilogue_rows<1, FAST>(acc, a, oc, pmult, pshift, phpot, pix_done, 32, lut, out);
      if (!more) break;
    }
  } else {
    for (; pb < n_pb;) {
      v16i acc[1];
      bias_acc(acc[0]);
      for (int t = 0; t < taps; ++t)
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afrag[t * 64], tap_load(t), acc[0], 0, 0, 0);
      if (ch_ok) epilogue_rows<1, FAST>(acc, a, oc, pmult, pshift, phpot, pix, 32, lut, out);
      advance();
    }
  }
}

// ---------------------------------------------------------------------------
// The same diagonal-MFMA depthwise for windows of at most 3 x 3 taps, laid out so that the
// vector ALU -- which the per-tap address arithmetic and the general epilogue of the kernel
// above keep busier than anything else on the large MobileNet layers -- is left with little
// more than the requantisation:
//   * a wave's 32 pixels are R whole row segments of W lanes (R * W <= 32) of one image
//     instead of 32 consecutive pixels of the flattened tensor: image, output rows and first
//     column of a block are wave-uniform (scalar registers), a lane's row and column within
//     the block never change, and a tap's address is one multiply-add per filter row;
//   * SHIFT (3 taps wide, stride 1, no dilation along W): a lane loads only the middle tap
//     of each filter row; the left and right taps are the same registers moved one lane up
//     or down the wave (DPP), so a block costs 3 loads instead of 9.  The first and last lane
//     of every row segment are halo: they load the neighbours' pixels, and what they compute
//     is not stored (W - 2 outputs per segment);
//   * accumulators start at zero and the bias rides in the 64-bit multiply-add of the
//     requantisation (requant_rows_c64; needs the layer's overflow-free form).
// A wave keeps its 32-channel block (nine A fragments in registers) and walks blocks.
// ---------------------------------------------------------------------------
struct DwRowsArgs {
  int rows, width, valid, halo;   // R, W, outputs per row segment (W - 2 * halo), 1 with SHIFT
  int xblocks, rblocks;           // column blocks per output row, row blocks per image (both below 2^15)
  int nblocks;                    // n * rblocks * xblocks
  // the walk, laid out by the host: blocks in flight per XCD, that step split into (image, row
  // block, column block) parts, and the first block of every XCD's run split the same way
  int nslots, d_n, d_rb, d_xb;
  int start_n[8], start_rb[8], start_xb[8];
  uint32_t magic_x, magic_r, magic_w;   // ceil(2^32 / d) of xblocks, rblocks, width: x / d == umulhi(x, magic), x, d < 2^16
};

template <bool SHIFT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(SHIFT ? 4 : 3, SHIFT ? 4 : 3))) void
conv_depthwise_rows_kernel(ConvArgs a, DwRowsArgs r) {
  __shared__ uint32_t lutw[64];
  __shared__ int32_t qlds[4][160];   // per wave: 32 (low, high) pairs of c64, then mult, shift, hpot of 32 channels
  gather_conv_args(a);
  gather_conv_args_more(a);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int p = lane & 31, fk = lane >> 5;
  const int n_cb = (a.ocw + 31) >> 5;
  // workgroups are dealt to the 8 XCDs round-robin; each XCD takes a contiguous run of blocks
  const int per_xcd = (r.nblocks + 7) >> 3;
  const int xcd = (int)(blockIdx.x & 7);
  const int b_end = min(r.nblocks, (xcd + 1) * per_xcd);
  const int gw = (int)(blockIdx.x >> 3) * 4 + wave;
  const int nslots = r.nslots;                              // blocks in flight per XCD (>= 1)
  // gw < 2^16 waves per XCD, n_cb < 2^16
  const int slot = n_cb == 1 ? gw : (int)__umulhi((uint32_t)gw, a.magic_c16);   // gw / n_cb (the host set magic_c16 for it)
  const int cb = gw - slot * n_cb;
  const bool relu = a.lo == 0;
  // Everything the wave fetches before its first block -- the parameters of its 32 channels, the
  // fused table, the filter fragments -- is requested in one go and parked afterwards: one trip
  // to memory, not one per array (a load under its own condition is waited for where it stands).
  // The parameter arrays are padded past the last channel block, so every lane may read them.
  const int32_t *c64 = relu ? a.qc64r : a.qc64;
  const int32_t qv0 = c64[2 * (cb * 32) + lane];
  const int32_t qv1 = a.qmult[cb * 32 + p], qv2 = a.qshift[cb * 32 + p], qv3 = a.qhpot[cb * 32 + p];
  uint32_t lutv = 0;
  if (a.has_lut && threadIdx.x < 64) lutv = a.lut.w[threadIdx.x];
  const int taps = a.kh * a.kw;
  const v4i *afrag = reinterpret_cast<const v4i *>(a.w) + (size_t)cb * taps * 64 + lane;
  v4i areg[3][3];
#pragma unroll
  for (int i = 0; i < 3; ++i)
#pragma unroll
    for (int j = 0; j < 3; ++j)
      areg[i][j] = (i < a.kh && j < a.kw) ? afrag[(i * a.kw + j) * 64] : v4i{0, 0, 0, 0};
  __builtin_amdgcn_sched_barrier(0);
  {
    int32_t *q = qlds[wave];
    q[lane] = qv0;
    q[64 + lane] = fk == 0 ? qv1 : qv2 - (relu ? 1 : 0);
    if (fk == 0) q[128 + lane] = qv3;
  }
  if (a.has_lut && threadIdx.x < 64) lutw[threadIdx.x] = lutv;
  __syncthreads();
  if (slot >= nslots) return;                               // no barrier below
  int b = xcd * per_xcd + slot;
  if (b >= b_end) return;
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  const int oc = cb * 32 + fk * 16;                         // this lane's 16 channels
  const bool ch_ok = oc < a.ocw;
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const int32_t *q = qlds[wave];
  const int32_t *pc64 = q + fk * 32, *pmult = q + 64 + fk * 16, *pshift = q + 96 + fk * 16, *phpot = q + 128 + fk * 16;

  // what never changes for a lane
  const int lr = (int)__umulhi((uint32_t)p, r.magic_w), lc = p - lr * r.width;
  const bool live = (p < r.rows * r.width) & ch_ok;
  const bool inner = live & (lc >= r.halo) & (lc < r.halo + r.valid);
  const int lrow_in = lr * a.sh;                            // input row offset of the lane's segment
  // column of the tap a lane loads first, relative to the block's first output column times sw:
  // SHIFT: the middle tap; otherwise the leftmost
  const int lcol_in = (lc - r.halo) * a.sw - a.pl + (SHIFT ? 1 : 0);
  const int row_bytes = a.iw * a.x_cs, drow_bytes = a.dh * row_bytes;

  // block -> (image, row block, column block), advanced by nslots blocks at a time
  int xb = r.start_xb[xcd] + slot;                          // slot < nslots <= 2^15
  // x / d by umulhi(x, ceil(2^32 / d)) is exact while x * d < 2^32; a divisor of 1 has no such constant
  int rb = r.start_rb[xcd] + (r.xblocks == 1 ? xb : (int)__umulhi((uint32_t)xb, r.magic_x));
  xb -= (rb - r.start_rb[xcd]) * r.xblocks;
  int n = r.start_n[xcd] + (r.rblocks == 1 ? rb : (int)__umulhi((uint32_t)rb, r.magic_r));
  rb -= (n - r.start_n[xcd]) * r.rblocks;
  const int d_xb = r.d_xb, d_rb = r.d_rb, d_n = r.d_n;

  uint32_t img_base = 0;                                    // scalar part of the addresses of the loads in flight
  auto request = [&](v4i (&bt)[3][3]) {
    const int ihb = rb * r.rows * a.sh - a.pt + lrow_in;    // first filter row's input row
    const int iw0 = xb * r.valid * a.sw + lcol_in;
    img_base = (uint32_t)n * (uint32_t)(a.ih * row_bytes);
    if (SHIFT) {
      const bool col_ok = live & ((unsigned)iw0 < (unsigned)a.iw);
      // rows and row pitch are below 2^23 (checked on the host); a first row above the image gives a
      // negative product, from which the rows below it are still reached
      const uint32_t off0 = (uint32_t)__mul24(ihb, row_bytes) + (uint32_t)(iw0 * a.x_cs + oc);
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const int ih = ihb + i * a.dh;
        const bool ok = col_ok & ((unsigned)ih < (unsigned)a.ih) & (i < a.kh);
        bt[i][1] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, ok ? off0 + (uint32_t)(i * drow_bytes) : kOobOffset,
                                                              img_base, 0);
      }
    } else {
      bool col_ok[3];
      uint32_t coff[3];
      const uint32_t off0 = (uint32_t)__mul24(ihb, row_bytes) + (uint32_t)(iw0 * a.x_cs + oc);
#pragma unroll
      for (int j = 0; j < 3; ++j) {
        const int iw = iw0 + j * a.dw;
        col_ok[j] = live & ((unsigned)iw < (unsigned)a.iw) & (j < a.kw);
        coff[j] = off0 + (uint32_t)(j * a.dw * a.x_cs);
      }
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        const int ih = ihb + i * a.dh;
        const bool row_ok = ((unsigned)ih < (unsigned)a.ih) & (i < a.kh);
#pragma unroll
        for (int j = 0; j < 3; ++j)
          bt[i][j] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
              xrsrc, (row_ok & col_ok[j]) ? coff[j] + (uint32_t)(i * drow_bytes) : kOobOffset, img_base, 0);
      }
    }
  };
  auto shift_lanes = [&](const v4i &m, int ctrl) {
    v4i o;
#pragma unroll
    for (int e = 0; e < 4; ++e)   // 0x138: wave_shr:1 (from lane l - 1), 0x130: wave_shl:1; the end lane reads 0
      o[e] = ctrl == 0 ? __builtin_amdgcn_mov_dpp(m[e], 0x138, 0xf, 0xf, true) : __builtin_amdgcn_mov_dpp(m[e], 0x130, 0xf, 0xf, true);
    return o;
  };

  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  v4i bt[3][3];
  request(bt);
  for (;;) {
    v16i acc[1];
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[0][e] = 0;
#pragma unroll
    for (int i = 0; i < 3; ++i) {
      if (SHIFT) {
        // lane l takes the left tap from lane l - 1 and the right tap from lane l + 1
        bt[i][0] = shift_lanes(bt[i][1], 0);
        bt[i][2] = shift_lanes(bt[i][1], 1);
      }
#pragma unroll
      for (int j = 0; j < 3; ++j)
        acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[i][j], bt[i][j], acc[0], 0, 0, 0);
    }
    // this block's output pixel, before the walk moves on
    const int oh = rb * r.rows + lr, ow = xb * r.valid + lc - r.halo;
    const bool st_ok = inner & (oh < a.oh) & (ow < a.ow);
    const int pix = (n * a.oh + oh) * a.ow + ow;
    b += nslots;
    xb += d_xb;
    if (xb >= r.xblocks) { xb -= r.xblocks; ++rb; }
    rb += d_rb;
    if (rb >= r.rblocks) { rb -= r.rblocks; ++n; }
    n += d_n;
    const bool more = b < b_end;
    if (more) request(bt);          // into the registers the MFMAs have just consumed
    uint32_t outw[1][4];
    if (relu) requant_rows_c64<1, true>(acc, 0, pc64, pmult, pshift, phpot, outw);
    else requant_rows_c64<1, false>(acc, a.lo, pc64, pmult, pshift, phpot, outw);
    if (st_ok) {
      const v4i o = {(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
      finish_chunk(o, o, (int64_t)pix * out.y_cs + oc, oc, a, out.y, lut);
    }
    if (!more) break;
  }
}

// ---------------------------------------------------------------------------
// The network stem: at most 4 input channels, so one pixel is one dword and the kw taps of
// a filter row are kw consecutive dwords of an input row.  A workgroup computes every
// output channel (at most 64) of 128 consecutive pixels of ONE output row.  The kh input
// rows that tile needs are fetched once with coalesced loads (lane = pixel), their first
// dword kept, and laid down in LDS as a compact patch [kh][column]; the MFMA B operand of
// filter row kh for output pixel p is then the 8 dwords from column p * sw of patch row kh
// (lane half h takes dwords 4h .. 4h+3): K = 32 bytes per filter row, taps kw .. 7 meeting
// zero weights.  No im2col gather from global memory, no address arithmetic per tap.  The
// filter (A operand, 16 bytes per lane per row and 32-channel block) stays in registers;
// the patch of the next tile is in flight while this one is multiplied and requantised.
// KH: filter rows held (kh <= KH); TM: 32-channel blocks (oc <= 32 * TM).  sw <= 2, kw <= 8.
// ---------------------------------------------------------------------------
constexpr int kStemPW = 264;   // patch row in dwords: 127 * 2 + 8, rounded up
// A wave takes all (at most two) 32-channel blocks of 32 pixels -- or, when the filter is
// too large to keep two blocks of it in registers at three waves per SIMD (7 rows, 64
// channels: 56 registers), one channel block of 64 pixels.
constexpr bool stem_split(int kh, int tm) { return kh * tm > 7; }
template <int KH, int TM, bool FAST>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(3, 3))) void
conv_stem_kernel(ConvArgs a) {
  constexpr int NLD = (KH * kStemPW + 255) / 256;
  constexpr bool SPLIT = stem_split(KH, TM);
  constexpr int NI = SPLIT ? 1 : TM;   // channel blocks per wave
  constexpr int NP = SPLIT ? 2 : 1;    // 32-pixel blocks per wave
  __shared__ uint32_t patch[2][KH * kStemPW];
  __shared__ uint32_t lutw[64];
  __shared__ int32_t qlds[4][TM * 32];   // bias, multiplier, rshift, 2^(rshift-1)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frow = lane & 31, fk = lane >> 5;
  const int ib = SPLIT ? (wave & 1) : 0;                  // first channel block of this wave
  const int pbase = SPLIT ? (wave >> 1) * 64 : wave * 32; // first pixel of this wave in the tile
  // parameters, table and filter fragments are requested together and parked afterwards (one
  // trip to memory; a thread holds one of the 4 * TM * 32 <= 256 parameter words)
  static_assert(4 * TM * 32 <= 256, "one parameter word per thread");
  int32_t qv = 0;
  const int qk = tid / (TM * 32), qc = tid - qk * (TM * 32);
  if (tid < 4 * TM * 32) {
    const int32_t *src = qk == 0 ? a.bias : qk == 1 ? a.qmult : qk == 2 ? a.qshift : a.qhpot;
    qv = src[qc];
  }
  uint32_t lutv = 0;
  if (a.has_lut && tid < 64) lutv = a.lut.w[tid];
  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;
  const OutRoute out{a.y, a.y_cs, a.lo, 0};

  v4i areg[NI][KH];
  {
    const v4i *afrag = reinterpret_cast<const v4i *>(a.w) + lane;
#pragma unroll
    for (int i = 0; i < NI; ++i)
#pragma unroll
      for (int r = 0; r < KH; ++r) areg[i][r] = afrag[((ib + i) * KH + r) * 64];
  }
  __builtin_amdgcn_sched_barrier(0);
  if (tid < 4 * TM * 32) qlds[qk][qc] = qv;
  if (a.has_lut && tid < 64) lutw[tid] = lutv;
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const int nseg = (a.ow + 127) >> 7;
  const int n_tiles = a.n * a.oh * nseg;
  const int used = a.kh * a.stem_pw;   // dwords of a patch that are read

  // workgroups are dealt to the 8 XCDs round-robin; each XCD takes a contiguous run of tiles
  // (consecutive output rows), so the input rows neighbouring tiles share meet in its L2
  const int per_xcd = (n_tiles + 7) >> 3, wg_stride = (int)(gridDim.x >> 3);
  const int tile_end = min(n_tiles, ((int)(blockIdx.x & 7) + 1) * per_xcd);
  int tile = (int)(blockIdx.x & 7) * per_xcd + (int)(blockIdx.x >> 3);
  if (tile >= tile_end) return;        // whole workgroup, before any barrier
  int n, oh, ow0;
  auto locate = [&](int t) {
    const int seg = t % nseg, r = t / nseg;
    oh = r % a.oh;
    n = r / a.oh;
    ow0 = seg << 7;
  };
  uint32_t stage[NLD];
  auto fetch = [&]() {
    const int ihb = oh * a.sh - a.pt, iwb = ow0 * a.sw - a.pl;
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      const int e = tid + q * 256;
      const int r = (int)(((uint32_t)e * a.magic_pw) >> 20);
      const int c = e - r * a.stem_pw;
      const int ih = ihb + r, iw = iwb + c;
      const bool ok = (e < used) & ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
      stage[q] = __builtin_amdgcn_raw_buffer_load_b32(
          xrsrc, ok ? (uint32_t)(((n * a.ih + ih) * a.iw + iw) * a.x_cs) : kOobOffset, 0, 0);
    }
  };
  auto deposit = [&](int buf) {
#pragma unroll
    for (int q = 0; q < NLD; ++q) {
      const int e = tid + q * 256;
      const int r = (int)(((uint32_t)e * a.magic_pw) >> 20);
      const int c = e - r * a.stem_pw;
      if (e < used) patch[buf][r * kStemPW + c] = stage[q];
    }
  };

  locate(tile);
  fetch();
  deposit(0);
  __syncthreads();
  int buf = 0;
  for (;;) {
    const int n_cur = n, oh_cur = oh, ow_cur = ow0;
    const int next = tile + wg_stride;
    const bool more = next < tile_end;
    if (more) {
      locate(next);
      fetch();
    }
    v16i acc[NI][NP];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int32_t *pb = &qlds[0][(ib + i) * 32 + fk * 16];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const v4i b = *reinterpret_cast<const v4i *>(pb + q * 4);
#pragma unroll
        for (int j = 0; j < NP; ++j) {
          acc[i][j][q * 4 + 0] = b[0]; acc[i][j][q * 4 + 1] = b[1];
          acc[i][j][q * 4 + 2] = b[2]; acc[i][j][q * 4 + 3] = b[3];
        }
      }
    }
    const uint32_t *prow = &patch[buf][(pbase + frow) * a.sw + fk * 4];
    const int pstep = 32 * a.sw;
#pragma unroll
    for (int r = 0; r < KH; ++r) {
#pragma unroll
      for (int j = 0; j < NP; ++j) {
        const uint32_t *src = prow + r * kStemPW + j * pstep;
        v4i b;
        b[0] = (int)src[0]; b[1] = (int)src[1]; b[2] = (int)src[2]; b[3] = (int)src[3];
#pragma unroll
        for (int i = 0; i < NI; ++i)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[i][r], b, acc[i][j], 0, 0, 0);
      }
    }
#pragma unroll
    for (int j = 0; j < NP; ++j) {
      const int ow = ow_cur + pbase + j * 32 + frow;
      const int pix = ow < a.ow ? (n_cur * a.oh + oh_cur) * a.ow + ow : a.npix;   // npix: nothing stored
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        const int oc = (ib + i) * 32 + fk * 16;
        if (oc < a.ocw) {
          const v16i one[1] = {acc[i][j]};
          epilogue_rows<1, FAST>(one, a, oc, &qlds[1][oc], &qlds[2][oc], &qlds[3][oc], pix, 32, lut, out);
        }
      }
    }
    if (!more) break;
    deposit(buf ^ 1);
    __syncthreads();   // the next patch is complete; everyone is done reading this one
    buf ^= 1;
    tile = next;
  }
}

// ---------------------------------------------------------------------------
// The stem with the max pool behind it (conv 7x7 / stride 2 + ReLU, pool 3x3 / stride 2: the
// head of the ImageNet networks) as one launch.  A workgroup of 8 waves owns `rows` pooled rows
// of one image over its whole width:
//   1. the input rows those need -- (2 * rows + 1 conv rows - 1) * sh + kh of them, one dword per
//      pixel, borders zero -- are fetched once into an LDS patch, every load in flight at once;
//   2. waves walk the tile's conv pixels (rows flattened) in blocks of 32: the MFMAs of
//      conv_stem_kernel (filter in registers, B operand = 8 consecutive patch dwords), the
//      two-instruction ReLU form of the requantisation, and the int8 results go to a conv tile in
//      LDS ([pixel][64 channels], rows padded to 72 bytes so that the 32 pixels of a block land in
//      different banks);
//   3. lanes take 8 channels of one pooled pixel: nine 8-byte LDS reads, the maximum with packed
//      16-bit unsigned ops on the even and odd bytes (values are 0..127 after the ReLU, so an empty
//      window position counts as 0), one 8-byte store -- 64 contiguous bytes per pixel.
// The conv result never travels to HBM and back (25.7 + 25.7 MB at ResNet-50's batch 32) unless
// the caller wants it (a.store_y: rows are then written from the LDS tile, whole lines).
// Needs: ReLU, the overflow-free requantisation, 33..64 output channels, 4..7 filter rows.
// ---------------------------------------------------------------------------
struct StemPoolArgs {
  int8_t *py;             // pooled result, channels-last
  int poh, pow, ppt, ppl, p_cs;
  int rows;               // pooled rows per tile
  int tiles_per_image, n_tiles;
  int crows;              // conv rows a tile holds: 2 * rows + 1
  int crows_last;         // ... the last tile of an image: down to the conv's last row, which a
                          // pool without bottom padding may not reach (the rows are still stored)
  int prows;              // patch rows of the larger of the two: (crows - 1) * sh + kh
  int pw;                 // patch row in dwords: (ow - 1) * sw + 8, rounded up to 4
  uint32_t magic_pw;      // ceil(2^32 / pw)
  uint32_t magic_pow;     // ceil(2^32 / pow)
};
constexpr int kStemPoolLoads = 20;     // patch dwords per lane at most (40 KiB of patch)
constexpr int kStemPoolCRow = 72;      // bytes of a conv-tile pixel row in LDS

__host__ __device__ inline unsigned stem_pool_lds_bytes(int prows, int pw, int cpix) {
  return (unsigned)(prows * pw * 4 + ((cpix * kStemPoolCRow + 15) & ~15));
}

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t x, uint32_t y) {
  return __builtin_bit_cast(uint32_t, __builtin_elementwise_max(__builtin_bit_cast(v2us, x),
                                                                __builtin_bit_cast(v2us, y)));
}

__global__ __launch_bounds__(512) void conv_stem_pool_kernel(ConvArgs a, StemPoolArgs s) {
  gather_conv_args(a);
  gather_conv_args_more(a);
  extern __shared__ __attribute__((aligned(16))) uint32_t sp_smem[];
  uint32_t *const patch = sp_smem;                                              // [prows][pw]
  int8_t *const ctile = reinterpret_cast<int8_t *>(patch + s.prows * s.pw);      // [crows * ow][72]
  const int cpix_max = max(s.crows, s.crows_last) * a.ow;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int frow = lane & 31, fk = lane >> 5;
  // a wave owns one half of the channels (32) and every fourth 32-pixel block.  The
  // requantisation constants of its lanes' 16 channels stay in registers: a lane requantises 16
  // values per 7 MFMAs, and fetching the parameters from LDS each time kept the LDS pipe busier
  // than the matrix pipe
  const int ih_ = wave & 1;                 // channel half
  const int lc = ih_ * 32 + fk * 16;        // first of this lane's 16 channels
  int64_t pc[16];
  int32_t pm[16], pr[16];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const v4i c01 = *reinterpret_cast<const v4i *>(a.qc64r + 2 * (lc + 4 * q));
    const v4i c23 = *reinterpret_cast<const v4i *>(a.qc64r + 2 * (lc + 4 * q) + 4);
    const v4i m4 = *reinterpret_cast<const v4i *>(a.qmult + lc + 4 * q);
    const v4i r4 = *reinterpret_cast<const v4i *>(a.qshift + lc + 4 * q);
    pc[4 * q + 0] = (int64_t)(((uint64_t)(uint32_t)c01[1] << 32) | (uint32_t)c01[0]);
    pc[4 * q + 1] = (int64_t)(((uint64_t)(uint32_t)c01[3] << 32) | (uint32_t)c01[2]);
    pc[4 * q + 2] = (int64_t)(((uint64_t)(uint32_t)c23[1] << 32) | (uint32_t)c23[0]);
    pc[4 * q + 3] = (int64_t)(((uint64_t)(uint32_t)c23[3] << 32) | (uint32_t)c23[2]);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      pm[4 * q + e] = m4[e];
      pr[4 * q + e] = r4[e] - 1;
    }
  }
  v4i areg[7];
  {
    const v4i *afrag = reinterpret_cast<const v4i *>(a.w) + lane;
#pragma unroll
    for (int r = 0; r < 7; ++r) areg[r] = afrag[(ih_ * 7 + r) * 64];
  }
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);

  for (int tile = (int)blockIdx.x; tile < s.n_tiles; tile += (int)gridDim.x) {
    const int n = tile / s.tiles_per_image;
    const int ti = tile - n * s.tiles_per_image;
    const int r0 = ti * s.rows;                               // first pooled row
    const int crows = ti == s.tiles_per_image - 1 ? s.crows_last : s.crows;
    const int cpix = crows * a.ow;
    const int nblk = (cpix + 31) >> 5;
    const int patch_dwords = ((crows - 1) * a.sh + a.kh) * s.pw;
    const int c0 = r0 * 2 - s.ppt;                            // first conv row held (-1 at a padded top)
    const int iy0 = c0 * a.sh - a.pt;                         // input row of patch row 0
    // ---- 1. the patch
    uint32_t stage[kStemPoolLoads];
#pragma unroll
    for (int q = 0; q < kStemPoolLoads; ++q) {
      const int e = tid + q * 512;
      const int j = (int)__umulhi((uint32_t)e, s.magic_pw);
      const int d = e - j * s.pw;
      const int iy = iy0 + j, ix = d - a.pl;
      const bool ok = (e < patch_dwords) & ((unsigned)iy < (unsigned)a.ih) & ((unsigned)ix < (unsigned)a.iw);
      stage[q] = __builtin_amdgcn_raw_buffer_load_b32(
          xrsrc, ok ? (uint32_t)(((n * a.ih + iy) * a.iw + ix) * a.x_cs) : kOobOffset, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < kStemPoolLoads; ++q) {
      const int e = tid + q * 512;
      if (e < patch_dwords) patch[e] = stage[q];
    }
    __syncthreads();
    // ---- 2. conv + ReLU requantisation into the LDS tile
    for (int b = wave >> 1; b < nblk; b += 4) {
      const int pl = b * 32 + frow;
      const int p = min(pl, cpix - 1);
      const int cr = (int)__umulhi((uint32_t)p, a.magic_ow);
      const int col = p - cr * a.ow;
      const uint32_t *prow = patch + (cr * a.sh) * s.pw + col * a.sw + fk * 4;
      v16i acc;
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[e] = 0;
      if (a.sw == 2) {
        // stride 2: a lane's four dwords start at an even dword (patch rows are a multiple of 4
        // dwords), so they are two 8-byte reads and the 64 lanes of one read cover 512
        // consecutive bytes -- no two lanes in one bank, where four dword reads put two
#pragma unroll
        for (int r = 0; r < 7; ++r) {
          const uint2 *src = reinterpret_cast<const uint2 *>(prow + r * s.pw);
          const uint2 lo = src[0], hi = src[1];
          const v4i bb = {(int)lo.x, (int)lo.y, (int)hi.x, (int)hi.y};
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[r], bb, acc, 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 7; ++r) {
          const uint32_t *src = prow + r * s.pw;
          v4i bb;
          bb[0] = (int)src[0]; bb[1] = (int)src[1]; bb[2] = (int)src[2]; bb[3] = (int)src[3];
          acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[r], bb, acc, 0, 0, 0);
        }
      }
      uint32_t outw[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        int32_t y[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // the ReLU form of requant_rows_c64: floor((acc * m + c) / 2^(31 + rshift)), clamped below
          const int64_t prod = (int64_t)acc[4 * q + e] * (int64_t)pm[4 * q + e] + pc[4 * q + e];
          y[e] = (int32_t)(prod >> 32) >> pr[4 * q + e];
        }
        outw[q] = pack_sat4(y[0], y[1], y[2], y[3], 0);
      }
      if (pl < cpix) {
        uint2 *dst = reinterpret_cast<uint2 *>(ctile + p * kStemPoolCRow + lc);
        dst[0] = uint2{outw[0], outw[1]};
        dst[1] = uint2{outw[2], outw[3]};
      }
    }
    __syncthreads();
    // ---- 3. the pooled rows (and, when asked for, the conv rows themselves)
    const int rows_here = min(s.rows, s.poh - r0);
    const int items = rows_here * s.pow * 8;
    for (int it = tid; it < items; it += 512) {
      const int cg = it & 7, pp = it >> 3;
      const int pr = (int)__umulhi((uint32_t)pp, s.magic_pow);
      const int pc = pp - pr * s.pow;
      // a window position outside the map is moved onto the nearest one inside, which the window
      // holds as well (every window starts inside the map): the maximum does not change.  The
      // 16-bit maximum of the raw words is right in its high bytes whatever the low bytes hold;
      // the low bytes take a second maximum over the masked words.
      int roff[3], coff[3];
#pragma unroll
      for (int d = 0; d < 3; ++d) {
        roff[d] = (min(max(c0 + 2 * pr + d, 0), a.oh - 1) - c0) * a.ow * kStemPoolCRow;
        coff[d] = min(max(2 * pc - s.ppl + d, 0), a.ow - 1) * kStemPoolCRow + cg * 8;
      }
      uint32_t e0 = 0, o0 = 0, e1 = 0, o1 = 0;
#pragma unroll
      for (int dy = 0; dy < 3; ++dy)
#pragma unroll
        for (int dx = 0; dx < 3; ++dx) {
          const uint2 v = *reinterpret_cast<const uint2 *>(ctile + roff[dy] + coff[dx]);
          e0 = pk_max_u16(e0, v.x & 0x00ff00ffu);
          o0 = pk_max_u16(o0, v.x);
          e1 = pk_max_u16(e1, v.y & 0x00ff00ffu);
          o1 = pk_max_u16(o1, v.y);
        }
      if (cg * 8 < s.p_cs)
        *reinterpret_cast<uint2 *>(s.py + ((int64_t)(n * s.poh + r0 + pr) * s.pow + pc) * s.p_cs + cg * 8) =
            uint2{e0 | (o0 & 0xff00ff00u), e1 | (o1 & 0xff00ff00u)};
    }
    if (a.store_y) {
      for (int it = tid; it < cpix * 8; it += 512) {
        const int cg = it & 7, p = it >> 3;
        const int cr = (int)__umulhi((uint32_t)p, a.magic_ow);
        const int col = p - cr * a.ow;
        if ((unsigned)(c0 + cr) < (unsigned)a.oh && cg * 8 < a.y_cs)
          *reinterpret_cast<uint2 *>(a.y + ((int64_t)(n * a.oh + c0 + cr) * a.ow + col) * a.y_cs + cg * 8) =
              *reinterpret_cast<const uint2 *>(ctile + p * kStemPoolCRow + cg * 8);
      }
    }
    // the next tile's patch goes into LDS nobody reads any more (the conv tile is read above, the
    // patch was last read before the barrier in front of this stage); its conv stage starts behind
    // the barrier that follows the patch stores, which every wave reaches only after this stage
  }
}

// ---------------------------------------------------------------------------
// MFMA kernel without LDS: every wave owns a tile of TM*32 output channels x
// TN*32 pixels and loads its MFMA operands straight from global memory in the
// fragment layout (lane l: row l & 31, bytes 16*(l >> 5) .. +15 of a 32-byte K
// slice), DEPTH K steps ahead in registers.  Waves never synchronise.  Weights are
// stored fragment by fragment so their loads are 1 KiB contiguous per wave;
// an activation load touches 32 bytes of 32 pixel rows.  Feeds the MFMAs at up to
// what the vector L1 delivers, which is all the small layers can use, at none of
// the LDS / barrier cost.
// ---------------------------------------------------------------------------
template <int TM, int TN, int DEPTH, int OCC, bool FAST, bool UNI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void
conv_mfma_reg_kernel(ConvArgs a) {
  gather_conv_args(a);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int logical_wg = (int)(blockIdx.x & 7) * a.tiles_per_xcd + (int)(blockIdx.x >> 3);
  const int wt = logical_wg * 4 + wave;        // this wave's tile; oc tiles of a pixel tile adjacent
  if (wt >= a.n_tiles) return;                 // no barriers anywhere below
  const int pix_tile = pixel_tile_of(a, wt);
  const int oc_tile = wt - pix_tile * a.n_oc_tiles;
  const int oc0 = oc_tile * (TM * 32);
  const OutRoute out = route_out(a, __builtin_amdgcn_readfirstlane(oc0));
  const int pix0 = pix_tile * (TN * 32);

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

  const int frow = lane & 31;
  const int fk = lane >> 5;
  const int nsteps = a.kp / 64;

  int poff[TN], ih0[TN], iw0[TN];
  const int ow_first = pix0 % a.ow;
  const int t_first = pix0 / a.ow;
  const int oh_first = t_first % a.oh;
  const int n_first = t_first / a.oh;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int delta = j * 32 + frow;
    const bool pv = pix0 + delta < a.npix;
    const uint32_t t1 = (uint32_t)(ow_first + delta);
    const uint32_t q1 = a.ow == 1 ? t1 : __umulhi(t1, a.magic_ow);
    const int ow = (int)(t1 - q1 * (uint32_t)a.ow);
    const uint32_t t2 = (uint32_t)oh_first + q1;
    const uint32_t q2 = a.oh == 1 ? t2 : __umulhi(t2, a.magic_oh);
    const int oh = (int)(t2 - q2 * (uint32_t)a.oh);
    const int n = n_first + (int)q2;
    ih0[j] = pv ? oh * a.sh - a.pt : -(1 << 28);
    iw0[j] = ow * a.sw - a.pl;
    poff[j] = ((n * a.ih + (oh * a.sh - a.pt)) * a.iw + iw0[j]) * a.x_cs + (UNI ? fk * 16 : 0);
    asm volatile("" : "+v"(poff[j]), "+v"(ih0[j]), "+v"(iw0[j]));
  }
  // weight fragments: [oc block of 32][K step][kk][lane] x 16 bytes
  uint32_t woff[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    woff[i] = (uint32_t)(((oc0 / 32 + i) * nsteps) * 2048 + lane * 16);
    asm volatile("" : "+v"(woff[i]));
  }

  v4i af[DEPTH][2][TM], bf[DEPTH][2][TN];

  auto load_step = [&](int slot, int step) {
    const bool in_k = step < nsteps;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[slot][kk][i] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
            wrsrc, in_k ? woff[i] : kOobOffset, step * 2048 + kk * 1024, 0);
    if (UNI) {
      const uint32_t kg0 = (uint32_t)(step * 4);
      const uint32_t tap = (kg0 * a.magic_c16) >> 20;
      const int cgrp0 = (int)(kg0 - tap * (uint32_t)a.c16);
      const int tkh = (int)((tap * a.magic_kw) >> 20);
      const int tkw = (int)tap - tkh * a.kw;
      const int dh_off = (int)kg0 < a.k16 ? tkh * a.dh : (1 << 28);
      const int dw_off = tkw * a.dw;
      const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp0 * 16;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int ih = ih0[j] + dh_off, iw = iw0[j] + dw_off;
        const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
        const uint32_t off = ok ? (uint32_t)(poff[j] + tap_off) : kOobOffset;
        bf[slot][0][j] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 0, 0);
        bf[slot][1][j] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 32, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const uint32_t kg = (uint32_t)(step * 4 + kk * 2 + fk);
        const uint32_t tap = (kg * a.magic_c16) >> 20;
        const int cgrp = (int)(kg - tap * (uint32_t)a.c16);
        const int tkh = (int)((tap * a.magic_kw) >> 20);
        const int tkw = (int)tap - tkh * a.kw;
        const int dh_off = (int)kg < a.k16 ? tkh * a.dh : (1 << 28);
        const int dw_off = tkw * a.dw;
        const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp * 16;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int ih = ih0[j] + dh_off, iw = iw0[j] + dw_off;
          const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
          bf[slot][kk][j] = buffer_load16(xrsrc, ok ? (uint32_t)(poff[j] + tap_off) : kOobOffset);
        }
      }
    }
  };

  // (the bias is requested, then the first K steps, and only then does it go into the accumulators:
  // one trip to memory before the first MFMA, not two)
  v16i acc[TM][TN];
  const int ocw0 = oc0 + fk * 16 * TM;
  v4i bias4[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const v4i *bp = reinterpret_cast<const v4i *>(a.bias + ocw0 + i * 16);
#pragma unroll
    for (int q = 0; q < 4; ++q) bias4[i][q] = bp[q];
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_step(d, d);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const v4i b = bias4[i][q];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j][q * 4 + 0] = b[0];
        acc[i][j][q * 4 + 1] = b[1];
        acc[i][j][q * 4 + 2] = b[2];
        acc[i][j][q * 4 + 3] = b[3];
      }
    }
  }

  auto mfma_step = [&](int slot) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[slot][kk][i], bf[slot][kk][j],
                                                            acc[i][j], 0, 0, 0);
  };
  // whole groups of DEPTH steps: branch-free body, ring slots are compile-time indices
  const int full = nsteps / DEPTH;
#pragma nounroll
  for (int g = 0; g < full; ++g) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      mfma_step(d);
      load_step(d, (g + 1) * DEPTH + d);
    }
  }
  // the last nsteps % DEPTH steps are already in the ring
  const int rem = nsteps - full * DEPTH;
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < rem) mfma_step(d);

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int oc = ocw0 + i * 16;
    if (oc < a.ocw)
      epilogue_rows<TN, FAST>(acc[i], a, oc, a.qmult + oc, a.qshift + oc, a.qhpot + oc, pix0 + frow, 32,
                              nullptr, out);
  }
}

// ---------------------------------------------------------------------------
// Split-K variant of the LDS-free kernel for layers with few output tiles and a
// long K (late 3x3 and reduction 1x1 layers): the four waves of a workgroup share
// one tile and take every fourth K step each, so four independent load -> MFMA
// chains run per tile; the partial sums meet once in LDS.
// ---------------------------------------------------------------------------
template <int TM, int TN, int DEPTH, int OCC, bool FAST, bool UNI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void
conv_mfma_splitk_kernel(ConvArgs a) {
  gather_conv_args(a);
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int logical_wg = (int)(blockIdx.x & 7) * a.tiles_per_xcd + (int)(blockIdx.x >> 3);
  const int wt = logical_wg;                   // the four waves share one tile and split K
  if (wt >= a.n_tiles) return;                 // uniform over the workgroup
  const int pix_tile = pixel_tile_of(a, wt);
  const int oc_tile = wt - pix_tile * a.n_oc_tiles;
  const int oc0 = oc_tile * (TM * 32);
  const OutRoute out = route_out(a, __builtin_amdgcn_readfirstlane(oc0));
  const int pix0 = pix_tile * (TN * 32);

  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);

  const int frow = lane & 31;
  const int fk = lane >> 5;
  const int nsteps_all = a.kp / 64;
  // wave w takes K steps w, w + 4, w + 8, ...
  const int nsteps = (nsteps_all - wave + 3) / 4;

  int poff[TN], ih0[TN], iw0[TN];
  const int ow_first = pix0 % a.ow;
  const int t_first = pix0 / a.ow;
  const int oh_first = t_first % a.oh;
  const int n_first = t_first / a.oh;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int delta = j * 32 + frow;
    const bool pv = pix0 + delta < a.npix;
    const uint32_t t1 = (uint32_t)(ow_first + delta);
    const uint32_t q1 = a.ow == 1 ? t1 : __umulhi(t1, a.magic_ow);
    const int ow = (int)(t1 - q1 * (uint32_t)a.ow);
    const uint32_t t2 = (uint32_t)oh_first + q1;
    const uint32_t q2 = a.oh == 1 ? t2 : __umulhi(t2, a.magic_oh);
    const int oh = (int)(t2 - q2 * (uint32_t)a.oh);
    const int n = n_first + (int)q2;
    ih0[j] = pv ? oh * a.sh - a.pt : -(1 << 28);
    iw0[j] = ow * a.sw - a.pl;
    poff[j] = ((n * a.ih + (oh * a.sh - a.pt)) * a.iw + iw0[j]) * a.x_cs + (UNI ? fk * 16 : 0);
    asm volatile("" : "+v"(poff[j]), "+v"(ih0[j]), "+v"(iw0[j]));
  }
  // weight fragments: [oc block of 32][K step][kk][lane] x 16 bytes
  uint32_t woff[TM];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    woff[i] = (uint32_t)(((oc0 / 32 + i) * nsteps_all) * 2048 + lane * 16);
    asm volatile("" : "+v"(woff[i]));
  }

  v4i af[DEPTH][2][TM], bf[DEPTH][2][TN];

  auto load_step = [&](int slot, int local_step) {
    const int step = local_step * 4 + wave;
    const bool in_k = step < nsteps_all;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < TM; ++i)
        af[slot][kk][i] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
            wrsrc, in_k ? woff[i] : kOobOffset, step * 2048 + kk * 1024, 0);
    if (UNI) {
      const uint32_t kg0 = (uint32_t)(step * 4);
      const uint32_t tap = (kg0 * a.magic_c16) >> 20;
      const int cgrp0 = (int)(kg0 - tap * (uint32_t)a.c16);
      const int tkh = (int)((tap * a.magic_kw) >> 20);
      const int tkw = (int)tap - tkh * a.kw;
      const int dh_off = (int)kg0 < a.k16 ? tkh * a.dh : (1 << 28);
      const int dw_off = tkw * a.dw;
      const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp0 * 16;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int ih = ih0[j] + dh_off, iw = iw0[j] + dw_off;
        const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
        const uint32_t off = ok ? (uint32_t)(poff[j] + tap_off) : kOobOffset;
        bf[slot][0][j] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 0, 0);
        bf[slot][1][j] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, off, 32, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const uint32_t kg = (uint32_t)(step * 4 + kk * 2 + fk);
        const uint32_t tap = (kg * a.magic_c16) >> 20;
        const int cgrp = (int)(kg - tap * (uint32_t)a.c16);
        const int tkh = (int)((tap * a.magic_kw) >> 20);
        const int tkw = (int)tap - tkh * a.kw;
        const int dh_off = (int)kg < a.k16 ? tkh * a.dh : (1 << 28);
        const int dw_off = tkw * a.dw;
        const int tap_off = (tkh * a.dh * a.iw + dw_off) * a.x_cs + cgrp * 16;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const int ih = ih0[j] + dh_off, iw = iw0[j] + dw_off;
          const bool ok = ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
          bf[slot][kk][j] = buffer_load16(xrsrc, ok ? (uint32_t)(poff[j] + tap_off) : kOobOffset);
        }
      }
    }
  };

  // the bias is requested, then the first K steps, and only then does the bias go into the
  // accumulators: taken the other way round the first operand loads leave after the bias has
  // come back, two trips to memory in a row
  v16i acc[TM][TN];
  const int ocw0 = oc0 + fk * 16 * TM;
  v4i bias4[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const v4i *bp = reinterpret_cast<const v4i *>(a.bias + ocw0 + i * 16);
#pragma unroll
    for (int q = 0; q < 4; ++q) bias4[i][q] = bp[q];
  }
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load_step(d, d);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v4i b = bias4[i][q];
      if (wave != 0) b = v4i{0, 0, 0, 0};
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j][q * 4 + 0] = b[0];
        acc[i][j][q * 4 + 1] = b[1];
        acc[i][j][q * 4 + 2] = b[2];
        acc[i][j][q * 4 + 3] = b[3];
      }
    }
  }

  auto mfma_step = [&](int slot) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[slot][kk][i], bf[slot][kk][j],
                                                            acc[i][j], 0, 0, 0);
  };
  // whole groups of DEPTH steps: branch-free body, ring slots are compile-time indices
  const int full = nsteps / DEPTH;
#pragma nounroll
  for (int g = 0; g < full; ++g) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      mfma_step(d);
      load_step(d, (g + 1) * DEPTH + d);
    }
  }
  // the last nsteps % DEPTH steps are already in the ring
  const int rem = nsteps - full * DEPTH;
#pragma unroll
  for (int d = 0; d < DEPTH - 1; ++d)
    if (d < rem) mfma_step(d);

  // reduce the four partial sums through LDS: block b = i * TN + j is summed and
  // finished (requantised, stored) by wave b % 4
  constexpr int NB = TM * TN;
  __shared__ v4i part[4 * NB * 4 * 64];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        v4i v = {acc[i][j][q * 4 + 0], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                 acc[i][j][q * 4 + 3]};
        part[((wave * NB + i * TN + j) * 4 + q) * 64 + lane] = v;
      }
  __syncthreads();
#pragma unroll
  for (int b = 0; b < NB; ++b) {
    if ((b & 3) != wave) continue;
    const int i = b / TN, j = b % TN;
    v16i sum[1];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      v4i t = part[((0 * NB + b) * 4 + q) * 64 + lane];
#pragma unroll
      for (int w = 1; w < 4; ++w) t += part[((w * NB + b) * 4 + q) * 64 + lane];
      sum[0][q * 4 + 0] = t[0];
      sum[0][q * 4 + 1] = t[1];
      sum[0][q * 4 + 2] = t[2];
      sum[0][q * 4 + 3] = t[3];
    }
    const int oc = ocw0 + i * 16;
    if (oc < a.ocw)
      epilogue_rows<1, FAST>(sum, a, oc, a.qmult + oc, a.qshift + oc, a.qhpot + oc,
                             pix0 + j * 32 + frow, 32, nullptr, out);
  }
}


// ---------------------------------------------------------------------------
// FullyConnected with few rows (the classifier of a network: 32 x 2048 -> 1000): one 32x32
// block of outputs per 32 output channels, and a K far too long for one wave per block to be
// anything but a chain of dependent loads.  So K is split over workgroups of ONE wave: wave
// (tile, split) multiplies its K range from operands fetched straight in MFMA layout (filter
// stored fragment by fragment, as for conv_mfma_reg_kernel) and leaves its 32x32 int32
// partial sum in a scratch buffer in device memory, [tile][split][lane][16]; a second launch
// -- the kernel boundary is what makes the partial sums of all XCDs visible, no fence or
// atomic is involved and no wave waits for another -- adds them and the bias, requantises
// and stores (ReLU before the requantisation, one multiplier / shift for the tensor:
// core/fullyconnected.cpp:64-87).
// ---------------------------------------------------------------------------
constexpr int kFcMaxTiles = 1024;                              // blocks of 32 x 32 outputs
constexpr size_t kFcPartialBytes = 64 * 16 * sizeof(int32_t);  // one wave's partial sum

__global__ __launch_bounds__(64) void fc_partial_kernel(ConvArgs a, v4i *parts, int splits, int steps_per_split) {
  const int lane = threadIdx.x;
  const int split = (int)blockIdx.x % splits;
  const int tile = (int)blockIdx.x / splits;        // pixel block * output-channel blocks + output-channel block
  const int ob = tile % a.n_oc_tiles, pb = tile / a.n_oc_tiles;
  const int nsteps = a.kp / 64;
  const int s0 = split * steps_per_split, s1 = min(nsteps, s0 + steps_per_split);
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
  const int frow = lane & 31, fk = lane >> 5;
  const int row = pb * 32 + frow;                   // "pixel" = row of the input matrix
  const uint32_t xoff = row < a.npix ? (uint32_t)(row * a.x_cs + fk * 16) : kOobOffset;
  const uint32_t woff = (uint32_t)(ob * nsteps) * 2048u + (uint32_t)lane * 16u;
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  for (int s = s0; s < s1; ++s) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const v4i af = (v4i)__builtin_amdgcn_raw_buffer_load_b128(wrsrc, woff, s * 2048 + kk * 1024, 0);
      const v4i bf = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, xoff, s * 64 + kk * 32, 0);
      acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, bf, acc, 0, 0, 0);
    }
  }
  v4i *mine = parts + ((size_t)(tile * splits + split) * 64 + lane) * 4;
#pragma unroll
  for (int q = 0; q < 4; ++q) mine[q] = v4i{acc[q * 4 + 0], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]};
}

// one workgroup per 32x32 block of outputs: wave q adds up dwords 4q .. 4q+3 of every lane's 16
// partial sums (eight loads in flight per lane), wave 0 collects the four quarters from LDS and
// runs the epilogue
template <bool FAST>
__global__ __launch_bounds__(256) void fc_reduce_kernel(ConvArgs a, const v4i *parts, int splits) {
  __shared__ v4i quarter[4][64];
  const int lane = threadIdx.x & 63, q = threadIdx.x >> 6;
  const int tile = (int)blockIdx.x;
  const int ob = tile % a.n_oc_tiles, pb = tile / a.n_oc_tiles;
  const int frow = lane & 31, fk = lane >> 5;
  const int oc = ob * 32 + fk * 16;                 // this lane's 16 channels
  const v4i *src = parts + ((size_t)tile * splits * 64 + lane) * 4 + q;
  v4i t = *reinterpret_cast<const v4i *>(a.bias + oc + q * 4);
  int sp = 0;
  for (; sp + 8 <= splits; sp += 8) {
    v4i v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[(size_t)(sp + u) * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) t += v[u];
  }
  for (; sp < splits; ++sp) t += src[(size_t)sp * 256];
  quarter[q][lane] = t;
  __syncthreads();
  if (q != 0) return;
  v16i sum[1];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const v4i r = quarter[k][lane];
    sum[0][k * 4 + 0] = r[0]; sum[0][k * 4 + 1] = r[1]; sum[0][k * 4 + 2] = r[2]; sum[0][k * 4 + 3] = r[3];
  }
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  if (oc < a.ocw)
    epilogue_rows<1, FAST>(sum, a, oc, a.qmult + oc, a.qshift + oc, a.qhpot + oc, pb * 32 + frow, 32, nullptr, out);
}

// The same product in ONE launch, for K of at least kFcOneWaves x 64: a workgroup of sixteen waves
// per 32x32 block of outputs, wave w multiplying K steps [w * spw, (w + 1) * spw) with the
// loads of two steps in flight at a time.  The sixteen partial sums meet in LDS (64 KiB,
// [wave][quarter][lane] of four dwords): every thread adds one quarter of four waves in place,
// wave 0 adds the four groups and the bias and runs the epilogue.  No scratch in device
// memory and no second launch, which on a classifier of 32 rows is most of the time.
constexpr int kFcOneWaves = 16;

template <bool FAST>
__global__ __launch_bounds__(64 * kFcOneWaves) void fc_one_kernel(ConvArgs a, int steps_per_wave) {
  __shared__ v4i part[kFcOneWaves * 4 * 64];
  gather_conv_args(a);
  gather_conv_args_more(a);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int tile = (int)blockIdx.x;
  const int ob = tile % a.n_oc_tiles, pb = tile / a.n_oc_tiles;
  const int nsteps = a.kp / 64;
  const int s0 = min(nsteps, wave * steps_per_wave), s1 = min(nsteps, s0 + steps_per_wave);
  const __amdgpu_buffer_rsrc_t xrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t wrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.w, 0, a.w_bytes, 0x00020000);
  const int frow = lane & 31, fk = lane >> 5;
  const int row = pb * 32 + frow;
  const uint32_t xoff = row < a.npix ? (uint32_t)(row * a.x_cs + fk * 16) : kOobOffset;
  const uint32_t woff = (uint32_t)(ob * nsteps) * 2048u + (uint32_t)lane * 16u;
  v16i acc;
#pragma unroll
  for (int e = 0; e < 16; ++e) acc[e] = 0;
  int s = s0;
  for (; s + 2 <= s1; s += 2) {
    v4i af[4], bf[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      af[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(wrsrc, woff, s * 2048 + u * 1024, 0);
      bf[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, xoff, s * 64 + u * 32, 0);
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[u], bf[u], acc, 0, 0, 0);
  }
  if (s < s1) {
    v4i af[2], bf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      af[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(wrsrc, woff, s * 2048 + u * 1024, 0);
      bf[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(xrsrc, xoff, s * 64 + u * 32, 0);
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[u], bf[u], acc, 0, 0, 0);
  }
#pragma unroll
  for (int q = 0; q < 4; ++q)
    part[(wave * 4 + q) * 64 + lane] = v4i{acc[q * 4 + 0], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]};
  __syncthreads();
  {
    // thread (group g of four waves, quarter q, lane): the sum lands where only it has read
    const int g = wave >> 2, q = wave & 3;
    v4i t = part[((g * 4 + 0) * 4 + q) * 64 + lane];
#pragma unroll
    for (int w = 1; w < 4; ++w) t += part[((g * 4 + w) * 4 + q) * 64 + lane];
    part[((g * 4) * 4 + q) * 64 + lane] = t;
  }
  __syncthreads();
  if (wave != 0) return;
  const int oc = ob * 32 + fk * 16;                 // this lane's 16 channels
  v16i sum[1];
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    v4i t = *reinterpret_cast<const v4i *>(a.bias + oc + q * 4);
#pragma unroll
    for (int g = 0; g < 4; ++g) t += part[((g * 4) * 4 + q) * 64 + lane];
    sum[0][q * 4 + 0] = t[0]; sum[0][q * 4 + 1] = t[1]; sum[0][q * 4 + 2] = t[2]; sum[0][q * 4 + 3] = t[3];
  }
  const OutRoute out{a.y, a.y_cs, a.lo, 0};
  if (oc < a.ocw)
    epilogue_rows<1, FAST>(sum, a, oc, a.qmult + oc, a.qshift + oc, a.qhpot + oc, pb * 32 + frow, 32, nullptr, out);
}

// The scratch of the allocation-free entry point: one array per device the library is loaded
// on.  Nothing in it has to start at zero: every partial sum the second launch reads was
// written by the first.
constexpr size_t kFcStaticPartials = 1024;          // (tile, split) pairs: 4 MiB of partial sums
constexpr size_t kFcStaticBytes = kFcStaticPartials * kFcPartialBytes;
static __device__ __align__(256) unsigned char scratch[kFcStaticBytes];
static void *g_static_scratch[64];                  // device address of `scratch`, per device
// who used a device's static scratch last: a call from another stream while that one's work is
// still in flight would race on the array and is refused
static std::mutex g_static_mu;
static const tpuhip_ctx *g_static_user[64];
static hipStream_t g_static_stream[64];

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
namespace {

struct TileCfg {
  int bm, bn, wm, wn;
  const char *name;
  int reg;   // 0: LDS kernel, one tile per workgroup; 1: the LDS-free kernel, bm x bn is the
             // tile of one wave; 2: its split-K form; 3: LDS kernel, persistent workgroups;
             // 4: patch kernel (bn = pixel slots of a tile of whole rows); 5: pointwise kernel;
             // 6: patch kernel, second form; 7: patch kernel, third form
  int bk;    // K bytes per step (pointwise kernel: the padded K it holds)
};

// The tile variants, in the order of their public index (conv desc algo = 16 + index).
// LDS kernels: X(index, name, persistent, BM, BN, WM, WN, BK, ring depth, waves per SIMD)
#define TPUHIP_LDS_TILES(X)                                     \
  X(0, "mfma_p_64x128", true, 64, 128, 2, 2, 64, 2, 3)          \
  X(1, "mfma_p_64x64", true, 64, 64, 2, 2, 64, 2, 4)            \
  X(2, "mfma_p_128x128", true, 128, 128, 2, 2, 64, 2, 2)        \
  X(3, "mfma_p_32x128", true, 32, 128, 1, 4, 64, 2, 3)          \
  X(4, "mfma_p_64x256", true, 64, 256, 1, 4, 64, 2, 1)          \
  X(5, "mfma_p_32x256", true, 32, 256, 1, 4, 64, 2, 2)          \
  X(6, "mfma_p_64x64_k128", true, 64, 64, 2, 2, 128, 2, 3)      \
  X(7, "mfma_p_64x64_k256", true, 64, 64, 2, 2, 256, 2, 2)      \
  X(8, "mfma_p_64x128_k128", true, 64, 128, 2, 2, 128, 2, 2)    \
  X(9, "mfma_64x64_k128", false, 64, 64, 2, 2, 128, 4, 0)       \
  X(10, "mfma_64x64_k256", false, 64, 64, 2, 2, 256, 2, 0)      \
  X(11, "mfma_64x128_k128", false, 64, 128, 2, 2, 128, 2, 0)    \
  X(12, "mfma_64x64_k128_d6", false, 64, 64, 2, 2, 128, 6, 0)
// LDS-free kernels: Y(index, name, split K, TM, TN, ring depth, waves per SIMD)
#define TPUHIP_REG_TILES(Y)                        \
  Y(13, "mfma_reg_32x64", false, 1, 2, 4, 3)       \
  Y(14, "mfma_reg_32x32", false, 1, 1, 4, 5)       \
  Y(15, "mfma_reg_64x64", false, 2, 2, 4, 2)       \
  Y(16, "mfma_splitk_64x64", true, 2, 2, 4, 2)     \
  Y(17, "mfma_splitk_32x64", true, 1, 2, 4, 3)

// patch kernels (3x3 / stride 1 / pad 1, input rows held in LDS): Z(index, name, BM, BN, BK, ring depth, waves per SIMD)
#define TPUHIP_PATCH_TILES(Z)                          \
  Z(18, "mfma_patch_64x128", 64, 128, 64, 2, 3)        \
  Z(19, "mfma_patch_64x256", 64, 256, 64, 2, 2)        \
  Z(20, "mfma_patch_64x128_k128", 64, 128, 128, 2, 2)  \
  Z(21, "mfma_patch_64x128_k256", 64, 128, 256, 2, 2)  \
  Z(22, "mfma_patch_64x64_k256", 64, 64, 256, 2, 2)

// pointwise kernels (1x1, unpadded, at most KP input channels, the filter slice resident in LDS):
// W(index, name, BM, BN, WM, WN, KP, staging buffers, waves per SIMD)
#define TPUHIP_PW_TILES(W)                                  \
  W(23, "mfma_pw_64x128_k64", 64, 128, 2, 2, 64, 2, 3)      \
  W(24, "mfma_pw_64x128_k128", 64, 128, 2, 2, 128, 2, 2)    \
  W(25, "mfma_pw_64x64_k256", 64, 64, 2, 2, 256, 2, 2)      \
  W(26, "mfma_pw_128x64_k64", 128, 64, 2, 2, 64, 2, 3)      \
  W(27, "mfma_pw_128x64_k128", 128, 64, 2, 2, 128, 2, 3)    \
  W(28, "mfma_pw_128x64_k256", 128, 64, 2, 2, 256, 1, 2)    \
  W(29, "mfma_pw_256x64_k64", 256, 64, 4, 1, 64, 2, 2)      \
  W(30, "mfma_pw_256x64_k128", 256, 64, 4, 1, 128, 1, 2)    \
  W(36, "mfma_pw_256x64_k64_w8", 256, 64, 4, 2, 64, 2, 4)   \
  W(37, "mfma_pw_256x64_k128_w8", 256, 64, 4, 2, 128, 1, 4) \
  W(38, "mfma_pw_128x64_k256_w8", 128, 64, 4, 2, 256, 1, 4) \
  W(39, "mfma_pw_64x128_k64_w8", 64, 128, 2, 4, 64, 2, 4)   \
  W(40, "mfma_pw_128x64_k64_w8", 128, 64, 4, 2, 64, 2, 4)   \
  W(59, "mfma_pw_96x128_k64", 96, 128, 1, 4, 64, 2, 3)

// row-patch kernels, second form (3x3 / stride 1 / pad 1, 64 to 1024 input channels, a power of two):
// V(index, name, BM, BN, WM, WN, BK, waves per SIMD)
#define TPUHIP_PATCH2_TILES(V)                          \
  V(31, "mfma_patch2_64x256", 64, 256, 1, 4, 256, 2)    \
  V(32, "mfma_patch2_64x128", 64, 128, 2, 2, 256, 2)    \
  V(33, "mfma_patch2_128x128", 128, 128, 2, 2, 128, 2)  \
  V(34, "mfma_patch2_64x64", 64, 64, 2, 2, 256, 2)      \
  V(35, "mfma_patch2_128x256", 128, 256, 2, 2, 128, 1)  \
  V(41, "mfma_patch2_64x256_w8", 64, 256, 2, 4, 256, 4) \
  V(42, "mfma_patch2_64x128_w8", 64, 128, 2, 4, 256, 4) \
  V(43, "mfma_patch2_128x128_w8", 128, 128, 4, 2, 128, 4) \
  V(44, "mfma_patch2_128x256_w8", 128, 256, 4, 2, 128, 2) \
  V(45, "mfma_patch2_32x256_w8", 32, 256, 1, 8, 256, 4) \
  V(46, "mfma_patch2_32x128", 32, 128, 1, 4, 256, 2) \
  V(47, "mfma_patch2_128x256_w8_k256", 128, 256, 4, 2, 256, 2) \
  V(48, "mfma_patch2_128x256_w8t_k256", 128, 256, 2, 4, 256, 2) \
  V(49, "mfma_patch2_128x256_w8t", 128, 256, 2, 4, 128, 2) \
  V(55, "mfma_patch2_256x256_w8", 256, 256, 2, 4, 128, 2) \
  V(56, "mfma_patch2_128x192_w8", 128, 192, 4, 2, 256, 2)

// row-patch kernels, third form (3x3 / stride 1 / pad 1, the four waves split K, 32 channels per
// workgroup, or 64: two channel blocks per wave): U3(index, name, pixel blocks of a pixel group, pixel groups, channel blocks)
#define TPUHIP_PATCH3_TILES(U3)               \
  U3(50, "mfma_patch3_32x128", 4, 1, 1)       \
  U3(51, "mfma_patch3_32x224", 7, 1, 1)       \
  U3(52, "mfma_patch3_32x256", 8, 1, 1)       \
  U3(53, "mfma_patch3_32x128_w8", 2, 2, 1)    \
  U3(54, "mfma_patch3_32x256_w8", 4, 2, 1)    \
  U3(57, "mfma_patch3_64x256_w8", 4, 2, 2)    \
  U3(58, "mfma_patch3_64x192_w8", 3, 2, 2)

struct TileTable {
  TileCfg t[64];
  int n = 0;
  TileTable() {
#define X(i, name, P, BM, BN, WM, WN, BK, D, O) \
  t[i] = TileCfg{BM, BN, WM, WN, name, P ? 3 : 0, BK}; \
  n = n > i ? n : i + 1;
    TPUHIP_LDS_TILES(X)
#undef X
#define Y(i, name, SPLIT, TM, TN, D, O) \
  t[i] = TileCfg{TM * 32, TN * 32, 1, 1, name, SPLIT ? 2 : 1, 64}; \
  n = n > i ? n : i + 1;
    TPUHIP_REG_TILES(Y)
#undef Y
#define Z(i, name, BM, BN, BK, D, O) \
  t[i] = TileCfg{BM, BN, 2, 2, name, 4, BK}; \
  n = n > i ? n : i + 1;
    TPUHIP_PATCH_TILES(Z)
#undef Z
#define W(i, name, BM, BN, WM, WN, KP, SD, O) \
  t[i] = TileCfg{BM, BN, WM, WN, name, 5, KP}; \
  n = n > i ? n : i + 1;
    TPUHIP_PW_TILES(W)
#undef W
#define V(i, name, BM, BN, WM, WN, BK, O) \
  t[i] = TileCfg{BM, BN, WM, WN, name, 6, BK}; \
  n = n > i ? n : i + 1;
    TPUHIP_PATCH2_TILES(V)
#undef V
#define U3(i, name, NB2, PW, OB) \
  t[i] = TileCfg{32 * OB, NB2 * PW * 32, 1, PW, name, 7, 64}; \
  n = n > i ? n : i + 1;
    TPUHIP_PATCH3_TILES(U3)
#undef U3
  }
};
const TileTable kTileTable;
const TileCfg *const kTiles = kTileTable.t;
inline int tile_bk(const TileCfg &t) { return t.bk; }
constexpr int kMaxTiles = 64;
#define kNumTiles (kTileTable.n)

template <bool SPLIT, int TM, int TN, int D, int O, bool FAST, bool UNI>
void launch_reg(tpuhip_ctx *ctx, dim3 grid, const ConvArgs &a) {
  if constexpr (SPLIT)
    launch(ctx, (conv_mfma_splitk_kernel<TM, TN, D, O, FAST, UNI>), grid, dim3(256), a);
  else
    launch(ctx, (conv_mfma_reg_kernel<TM, TN, D, O, FAST, UNI>), grid, dim3(256), a);
}

// the patch kernel's LDS patch is dynamic: (rows + 2) x (W + 2) x C bytes of this layer
// Raises a kernel's dynamic LDS limit, once per kernel and size (kernels of one signature share
// their function-pointer type, so the record is keyed by the kernel's address); on failure the
// runtime's last error stays set for the caller to report.
bool raise_lds_limit(const void *kernel, unsigned bytes) {
  static std::mutex mu;
  static std::map<const void *, unsigned> raised;
  std::lock_guard<std::mutex> lock(mu);
  auto it = raised.find(kernel);
  if (it != raised.end() && it->second >= bytes) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return false;
  raised[kernel] = bytes;
  return true;
}

template <typename F>
void launch_patch(tpuhip_ctx *ctx, F kernel, dim3 grid, const ConvArgs &a, bool dynamic, unsigned stage_bytes) {
  if (dynamic) (void)raise_lds_limit((const void *)kernel, kPatchBytesDyn);
  // the patch, or the staged output tile that takes its place in the epilogue if that is larger
  const unsigned smem = dynamic ? std::max((unsigned)((a.pstep_pix + 2) * a.stem_pw * (a.c16 * 16)), stage_bytes) : 0u;
  if (ctx->prof_start)
    hipExtLaunchKernelGGL(kernel, grid, dim3(256), smem, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a);
  else
    hipLaunchKernelGGL(kernel, grid, dim3(256), smem, ctx->stream, a);
}

// dynamic LDS of a pointwise tile variant: filter slice, two pixel tiles, the staged output
// tile(s), five parameter planes, the fused table
constexpr unsigned pw_lds_bytes(int bm, int bn, int kp, int sd) {
  return (unsigned)(bm * kp + 2 * bn * kp + sd * bn * (bm + 16) + 5 * bm * 4 + 256);
}

template <typename F>
bool pw_prepare(F kernel, unsigned lds) {
  return raise_lds_limit((const void *)kernel, lds);
}

void launch_pw(tpuhip_ctx *ctx, int tile, dim3 grid, const ConvArgs &a) {
  switch (tile) {
#define W(i, name, BM, BN, WM, WN, KP, SD, O)                                                           \
  case i: {                                                                                             \
    auto kernel = conv_pw_kernel<BM, BN, WM, WN, KP, SD, O>;                                            \
    constexpr unsigned lds = pw_lds_bytes(BM, BN, KP, SD);                                              \
    if (!pw_prepare(kernel, lds)) break;                                                                \
    if (ctx->prof_start)                                                                                \
      hipExtLaunchKernelGGL(kernel, grid, dim3(WM * WN * 64), lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                \
      hipLaunchKernelGGL(kernel, grid, dim3(WM * WN * 64), lds, ctx->stream, a);                        \
  } break;
    TPUHIP_PW_TILES(W)
#undef W
  }
}

// workgroups of pointwise tile variant `tile` that fit on one CU at once
int pw_occupancy(int tile) {
  int n = 0;
  hipError_t e = hipErrorInvalidValue;
  switch (tile) {
#define W(i, name, BM, BN, WM, WN, KP, SD, O)                                                           \
  case i:                                                                                               \
    if (pw_prepare(conv_pw_kernel<BM, BN, WM, WN, KP, SD, O>, pw_lds_bytes(BM, BN, KP, SD)))             \
      e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, conv_pw_kernel<BM, BN, WM, WN, KP, SD, O>, WM * WN * 64, \
                                                       pw_lds_bytes(BM, BN, KP, SD));                   \
    break;
    TPUHIP_PW_TILES(W)
#undef W
  }
  if (e != hipSuccess) (void)hipGetLastError();
  return e == hipSuccess && n > 0 ? n : 1;
}

// ---- row-patch kernels, second form
constexpr int kPatch2MaxChunks = 18 * 256;     // 16-byte input chunks a workgroup's patch may hold
constexpr int kLdsBytes = 160 * 1024;

inline unsigned patch2_lds_bytes(const TileCfg &c, int th, int ow, int ic) {
  return (unsigned)(5 * c.bm * 4 + 256 + 2 * c.bm * (c.bk + 16) + (th + 2) * ((ow + 2) * (ic + 16) + kPatch2RowPad));
}

// rows of one image a tile holds; 0: the layer does not fit this kernel
int patch2_rows(const tpuhip_conv_desc &d, const TileCfg &c) {
  const bool shape_ok = d.g == 1 && d.kh == 3 && d.kw == 3 && d.sh == 1 && d.sw == 1 && d.dh == 1 && d.dw == 1 &&
                        d.pt == 1 && d.pb == 1 && d.pl == 1 && d.pr == 1 && !d.ins_h && !d.ins_w && !d.relu_first &&
                        d.oh == d.ih && d.ow == d.iw && d.x_cs == d.ic && d.ic >= 64 && d.ic <= 1024 &&
                        (d.ic & (d.ic - 1)) == 0;
  if (!shape_ok || d.ow > c.bn) return 0;
  int th = std::min(c.bn / d.ow, d.oh);
  while (th >= 1 && ((th + 2) * (d.ow + 2) * (d.ic / 16) > kPatch2MaxChunks ||
                     patch2_lds_bytes(c, th, d.ow, d.ic) > (unsigned)kLdsBytes))
    --th;
  if (th < 1) return 0;
  const int tiles = (d.oh + th - 1) / th;      // evened out over the image
  return (d.oh + tiles - 1) / tiles;
}

void launch_patch2(tpuhip_ctx *ctx, int tile, dim3 grid, const ConvArgs &a, unsigned lds) {
  switch (tile) {
#define V(i, name, BM, BN, WM, WN, BK, O)                                                               \
  case i: {                                                                                             \
    auto kernel = conv_patch2_kernel<BM, BN, WM, WN, BK, O>;                                            \
    if (!pw_prepare(kernel, (unsigned)kLdsBytes)) break;                                                \
    if (ctx->prof_start)                                                                                \
      hipExtLaunchKernelGGL(kernel, grid, dim3(WM * WN * 64), lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                \
      hipLaunchKernelGGL(kernel, grid, dim3(WM * WN * 64), lds, ctx->stream, a);                        \
  } break;
    TPUHIP_PATCH2_TILES(V)
#undef V
  }
}

// ---- row-patch kernels, third form
struct Patch3Plan {
  int th = 0;      // rows of a tile (0: the layer does not fit this kernel)
  int imgs = 1;    // whole images per tile
  unsigned lds = 0;
};

Patch3Plan patch3_plan(const tpuhip_conv_desc &d, const TileCfg &c) {
  Patch3Plan pl;
  const bool shape_ok = d.g == 1 && d.kh == 3 && d.kw == 3 && d.sh == 1 && d.sw == 1 && d.dh == 1 && d.dw == 1 &&
                        d.pt == 1 && d.pb == 1 && d.pl == 1 && d.pr == 1 && !d.ins_h && !d.ins_w && !d.relu_first &&
                        d.oh == d.ih && d.ow == d.iw && d.x_cs == d.ic && d.ic >= 64 && d.ic <= 1024 &&
                        (d.ic & (d.ic - 1)) == 0;
  if (!shape_ok || d.ow > c.bn) return pl;
  const int nblk = c.bn / 32;
  auto lds_bytes = [&](int th, int imgs) {
    const int64_t patch = (int64_t)imgs * (th + 2) * ((d.ow + 2) * (d.ic + 16) + kPatch2RowPad);
    const int64_t red = (int64_t)nblk * 3 * 4096, stage = (int64_t)c.bn * (c.bm + 16);
    return (int64_t)(5 * c.bm * 4 + 256) + std::max(patch, std::max(red, stage));
  };
  int imgs = std::min(d.n, c.bn / (d.oh * d.ow));
  while (imgs > 1 && lds_bytes(d.oh, imgs) > kLdsBytes) --imgs;
  if (imgs > 1) {
    // whole images: evened out over the batch
    const int tiles = (d.n + imgs - 1) / imgs;
    pl.imgs = (d.n + tiles - 1) / tiles;
    pl.th = d.oh;
  } else {
    int th = std::min(c.bn / d.ow, d.oh);
    while (th >= 1 && lds_bytes(th, 1) > kLdsBytes) --th;
    if (th < 1) return pl;
    const int tiles = (d.oh + th - 1) / th;      // evened out over the image
    pl.th = (d.oh + tiles - 1) / tiles;
  }
  pl.lds = (unsigned)lds_bytes(pl.th, pl.imgs);
  return pl;
}

void launch_patch3(tpuhip_ctx *ctx, int tile, dim3 grid, const ConvArgs &a, unsigned lds) {
  switch (tile) {
#define U3(i, name, NB2, PW, OB)                                                                        \
  case i: {                                                                                             \
    auto kernel = conv_patch3_kernel<NB2, PW, OB>;                                                      \
    if (!pw_prepare(kernel, (unsigned)kLdsBytes)) break;                                                \
    if (ctx->prof_start)                                                                                \
      hipExtLaunchKernelGGL(kernel, grid, dim3(256 * PW), lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                \
      hipLaunchKernelGGL(kernel, grid, dim3(256 * PW), lds, ctx->stream, a);                            \
  } break;
    TPUHIP_PATCH3_TILES(U3)
#undef U3
  }
}

template <bool FAST, int MODE>
void launch_mfma(tpuhip_ctx *ctx, int tile, dim3 grid, const ConvArgs &a) {
  constexpr bool UNI = MODE == kModeUniform;
  switch (tile) {
#define X(i, name, P, BM, BN, WM, WN, BK, D, O)                                             \
  case i:                                                                                   \
    launch(ctx, (conv_mfma_kernel<BM, BN, WM, WN, BK, D, O, P, FAST, MODE>), grid,          \
           dim3(WM * WN * 64), a);                                                          \
    break;
    TPUHIP_LDS_TILES(X)
#undef X
#define Y(i, name, SPLIT, TM, TN, D, O) \
  case i: launch_reg<SPLIT, TM, TN, D, O, FAST, UNI>(ctx, grid, a); break;
    TPUHIP_REG_TILES(Y)
#undef Y
#define Z(i, name, BM, BN, BK, D, O) \
  case i: launch_patch(ctx, (conv_patch_kernel<BM, BN, BK, D, O, FAST>), grid, a, BK == 256, BN * stage_row_bytes<BM>()); break;
    TPUHIP_PATCH_TILES(Z)
#undef Z
  }
}

// workgroups of LDS tile variant `tile` that fit on one CU at once
template <bool FAST, int MODE>
int persist_occupancy(int tile) {
  int n = 0;
  hipError_t e = hipErrorInvalidValue;
  switch (tile) {
#define X(i, name, P, BM, BN, WM, WN, BK, D, O)                                              \
  case i:                                                                                    \
    e = hipOccupancyMaxActiveBlocksPerMultiprocessor(                                        \
        &n, conv_mfma_kernel<BM, BN, WM, WN, BK, D, O, P, FAST, MODE>, WM * WN * 64, 0);     \
    break;
    TPUHIP_LDS_TILES(X)
#undef X
  }
  if (e != hipSuccess) (void)hipGetLastError();   // clear it: the caller falls back to 1
  return e == hipSuccess && n > 0 ? n : 1;
}

// the (FAST, MODE) instantiation a prepacked conv dispatches to
int conv_mode(const tpuhip_conv_weights *w) {
  const bool uni = (w->c16 % (tile_bk(kTiles[w->tile]) / 16)) == 0;
  return w->smallc ? kModeSmallC : uni ? kModeUniform : kModeGeneral;
}

int persist_wgs_per_cu(const tpuhip_conv_weights *w) {
  // 0 = not asked yet.  Contexts on several host threads may ask at once: every writer
  // stores the same value, so relaxed atomics are all that is needed.
  static std::atomic<int> cache[kMaxTiles][2][3];
  const int mode = kTiles[w->tile].reg == 5 ? 0 : conv_mode(w);
  std::atomic<int> &slot = cache[w->tile][w->fast ? 1 : 0][mode];
  int c = slot.load(std::memory_order_relaxed);
  if (c == 0) {
    if (kTiles[w->tile].reg == 5)
      c = pw_occupancy(w->tile);
    else if (w->fast)
      c = mode == kModeSmallC ? persist_occupancy<true, kModeSmallC>(w->tile)
          : mode == kModeUniform ? persist_occupancy<true, kModeUniform>(w->tile)
                                 : persist_occupancy<true, kModeGeneral>(w->tile);
    else
      c = mode == kModeSmallC ? persist_occupancy<false, kModeSmallC>(w->tile)
          : mode == kModeUniform ? persist_occupancy<false, kModeUniform>(w->tile)
                                 : persist_occupancy<false, kModeGeneral>(w->tile);
    slot.store(c, std::memory_order_relaxed);
  }
  return c;
}

// Default tile when the variants are not timed on first use: the persistent tiles,
// narrow in output channels for thin layers, wide in pixels when there are enough of
// them to give every CU several tiles.
int pick_tile(const tpuhip_conv_desc &d, int k16, int num_cu) {
  (void)k16;
  const int64_t npix = (int64_t)d.n * d.oh * d.ow;
  if (d.oc <= 32) return 3;
  const int64_t tiles128 = ceil_div64(npix, 128) * ceil_div64(d.oc, 64);
  return tiles128 >= 2 * (int64_t)num_cu ? 0 : 1;
}

int check_desc(const tpuhip_conv_desc &d) {
  TPUHIP_REQUIRE(d.n > 0 && d.ic > 0 && d.ih > 0 && d.iw > 0 && d.oc > 0 && d.oh > 0 && d.ow > 0,
                 "conv: non-positive dimension");
  TPUHIP_REQUIRE(d.g > 0 && d.ic % d.g == 0 && d.oc % d.g == 0, "conv: bad group count %d", d.g);
  TPUHIP_REQUIRE(d.kh > 0 && d.kw > 0 && d.sh > 0 && d.sw > 0 && d.dh > 0 && d.dw > 0,
                 "conv: bad kernel/stride/dilation");
  TPUHIP_REQUIRE(d.pt >= 0 && d.pb >= 0 && d.pl >= 0 && d.pr >= 0 && d.ins_h >= 0 && d.ins_w >= 0,
                 "conv: negative padding");
  // an input of at most 4 channels may lie one dword per pixel (the stem path reads it that way)
  TPUHIP_REQUIRE(d.x_cs >= d.ic && d.y_cs >= d.oc && (d.x_cs % 16 == 0 || d.x_cs == 4) && d.y_cs % 16 == 0,
                 "conv: channel strides must be multiples of 16 covering the channels "
                 "(x_cs %d ic %d, y_cs %d oc %d)", d.x_cs, d.ic, d.y_cs, d.oc);
  const int ihd = (d.ih - 1) * (d.ins_h + 1) + 1, iwd = (d.iw - 1) * (d.ins_w + 1) + 1;
  const int oh = (ihd + d.pt + d.pb - (d.dh * (d.kh - 1) + 1)) / d.sh + 1;
  const int ow = (iwd + d.pl + d.pr - (d.dw * (d.kw - 1) + 1)) / d.sw + 1;
  // the reference's importers may round up (Caffe ceil mode) by padding b/r; all
  // that matters for memory safety is that every output maps to a legal window
  TPUHIP_REQUIRE(d.oh <= oh && d.ow <= ow, "conv: output %dx%d larger than the window grid %dx%d",
                 d.oh, d.ow, oh, ow);
  // the kernels index pixels and input bytes with 32-bit integers
  TPUHIP_REQUIRE(d.oh < 65536 && d.ow < 65536 && (int64_t)d.n * d.oh * d.ow < (1ll << 30) &&
                     (int64_t)d.n * (d.ih + d.pt + d.pb + 2) * (d.iw + d.pl + d.pr + 2) * d.x_cs <
                         (1ll << 31) &&
                     (int64_t)d.n * d.oh * d.ow * d.y_cs < (1ll << 40),
                 "conv: tensor too large");
  return TPUHIP_OK;
}

// (re)builds the device filter of an MFMA conv for tile variant `tile`
int pack_mfma_weights(tpuhip_ctx *ctx, tpuhip_conv_weights *cw, int tile) {
  const tpuhip_conv_desc &d = cw->d;
  const TileCfg &t = kTiles[tile];
  const int tm = t.bm / t.wm / 32;
  const int icp = round_up(d.ic, 16);
  const int ocp = round_up(d.oc, t.bm);
  cw->smallc = d.ic <= 4 && (t.reg == 0 || t.reg == 3);
  cw->c16 = icp / 16;
  cw->k16 = cw->smallc ? (d.kh * d.kw * 4 + 15) / 16 : d.kh * d.kw * cw->c16;
  cw->kp = round_up(cw->k16 * 16, tile_bk(t));
  if (t.reg == 5 && cw->kp != t.bk) return set_error(TPUHIP_ERR_INVALID, "conv: tile %s holds %d input channels", t.name, t.bk);
  std::vector<int8_t> packed((size_t)ocp * cw->kp, 0);
  const int8_t *filter = cw->host_filter.data();
  std::vector<int8_t> rowbuf((size_t)cw->kp);
  const int nsteps = cw->kp / 64;
  for (int row = 0; row < ocp; ++row) {
    const int tile0 = row / t.bm * t.bm;
    const int oc = tile0 + mfma_row_to_oc(row - tile0, tm);
    if (oc >= d.oc) continue;
    std::fill(rowbuf.begin(), rowbuf.end(), 0);
    const int8_t *src = filter + (size_t)oc * d.ic * d.kh * d.kw;
    const int kstride = cw->smallc ? 4 : icp;   // channels per tap in the K order
    for (int c = 0; c < d.ic; ++c)
      for (int k = 0; k < d.kh * d.kw; ++k)
        rowbuf[(size_t)k * kstride + c] = src[(size_t)c * d.kh * d.kw + k];
    if (t.reg == 0 || t.reg == 3 || t.reg == 4) {
      memcpy(packed.data() + (size_t)row * cw->kp, rowbuf.data(), rowbuf.size());
    } else if (t.reg == 6) {
      // [output-channel tile][K step][row][BK bytes]: every step's tile is contiguous
      const int r = row - tile0;
      int8_t *img = packed.data() + (size_t)(tile0 / t.bm) * t.bm * cw->kp;
      for (int st = 0; st < cw->kp / t.bk; ++st)
        memcpy(img + ((size_t)st * t.bm + r) * t.bk, rowbuf.data() + (size_t)st * t.bk, t.bk);
    } else if (t.reg == 5) {
      // the LDS image of every output-channel tile: [64-byte K chunk][row][4 x 16 bytes], the
      // 16-byte position XORed with (row >> 2) & 3
      const int r = row - tile0;
      int8_t *img = packed.data() + (size_t)(tile0 / t.bm) * t.bm * cw->kp;
      for (int kc = 0; kc < cw->kp / 64; ++kc)
        for (int c4 = 0; c4 < 4; ++c4)
          memcpy(img + ((size_t)(kc * t.bm + r) * 4 + (c4 ^ ((r >> 2) & 3))) * 16,
                 rowbuf.data() + (size_t)kc * 64 + c4 * 16, 16);
    } else {
      // fragment order: [row / 32][K step][kk][lane = (row & 31) + 32 * half][16 bytes]
      const int blk = row / 32, r = row % 32;
      for (int step = 0; step < nsteps; ++step)
        for (int kk = 0; kk < 2; ++kk)
          for (int half = 0; half < 2; ++half)
            memcpy(packed.data() + ((size_t)(blk * nsteps + step) * 2 + kk) * 1024 +
                       (size_t)(r + 32 * half) * 16,
                   rowbuf.data() + (size_t)step * 64 + (kk * 2 + half) * 16, 16);
    }
  }
  if (cw->w) {
    if (int rc = tpuhip_free(ctx, cw->w)) return rc;
    cw->w = nullptr;
  }
  if (int rc = tpuhip_malloc(ctx, packed.size(), (void **)&cw->w)) return rc;
  if (int rc = tpuhip_upload(ctx, cw->w, packed.data(), packed.size())) return rc;
  cw->tile = tile;
  cw->ocp = ocp;
  return TPUHIP_OK;
}

// the fused table lives in the LDS of the LDS kernels
bool tile_has_lds_epilogue(int t) {
  return kTiles[t].reg == 0 || kTiles[t].reg == 3 || kTiles[t].reg == 5 || kTiles[t].reg == 6 || kTiles[t].reg == 7;
}

// the pointwise kernels: 1x1 window, no padding, no dilation (any stride), the input channels
// within the K the variant holds (and more than half of it, or the smallest variant)
bool pw_shape_ok(const tpuhip_conv_desc &d, const TileCfg &c) {
  const int icp = round_up(d.ic, 16);
  return d.g == 1 && d.kh == 1 && d.kw == 1 && d.pt == 0 && d.pl == 0 && d.pb == 0 && d.pr == 0 && !d.ins_h &&
         !d.ins_w && !d.relu_first && icp <= c.bk && (c.bk == 64 || icp > c.bk / 2) && d.ic > 4;
}

// rows of one image a patch tile holds; 0: the layer does not fit the patch kernel
int patch_rows(const tpuhip_conv_desc &d, const TileCfg &c) {
  const bool shape_ok = d.g == 1 && d.kh == 3 && d.kw == 3 && d.sh == 1 && d.sw == 1 && d.dh == 1 && d.dw == 1 &&
                        d.pt == 1 && d.pb == 1 && d.pl == 1 && d.pr == 1 && !d.ins_h && !d.ins_w &&
                        d.oh == d.ih && d.ow == d.iw && d.x_cs == d.ic &&
                        (d.ic == 64 || d.ic == 128 || d.ic == 256 || d.ic == 512) && d.ic % c.bk == 0;
  if (!shape_ok || d.ow > c.bn) return 0;
  // as many rows as the pixel slots and the patch buffer allow, then evened out over the image
  const int fit = (int)((c.bk == 256 ? kPatchBytesDyn : kPatchBytes) / ((int64_t)(d.ow + 2) * d.ic)) - 2;
  const int th_max = std::min(std::min(c.bn / d.ow, d.oh), fit);
  if (th_max < 1) return 0;
  const int tiles = (d.oh + th_max - 1) / th_max;
  return (d.oh + tiles - 1) / tiles;
}

bool tile_is_candidate(const tpuhip_conv_desc &d, int t) {
  const TileCfg &c = kTiles[t];
  if (c.reg == 4 && patch_rows(d, c) == 0) return false;
  if (c.reg == 5 && !pw_shape_ok(d, c)) return false;
  if (c.reg == 6 && patch2_rows(d, c) == 0) return false;
  if (c.reg == 7) return patch3_plan(d, c).th > 0;
  if (d.ic <= 4 && (c.reg == 1 || c.reg == 2)) return false;   // prefer the 4-channel K packing of the LDS kernels
  return !(c.bm > 32 && c.bm / 2 >= round_up(d.oc, 32));   // more than half the rows idle
}

void fill_args(const tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
               ConvArgs *out) {
  const tpuhip_conv_desc &d = w->d;
  ConvArgs a{};
  a.x = (const int8_t *)x;
  a.w = w->w;
  a.bias = w->bias;
  a.qp = w->qp;
  a.qmult = w->qplanes;
  a.qshift = w->qplanes + w->nparam;
  a.qhpot = w->qplanes + 2 * w->nparam;
  a.qc64 = w->qc64;
  a.qc64r = w->qc64 + 2 * w->nparam;
  a.y = (int8_t *)y;
  a.n = d.n; a.ih = d.ih; a.iw = d.iw; a.x_cs = d.x_cs;
  a.oh = d.oh; a.ow = d.ow; a.y_cs = d.y_cs;
  a.oc = d.oc; a.ocw = round_up(d.oc, 16); a.icg = d.ic / d.g; a.ocg = d.oc / d.g; a.g = d.g;
  a.kh = d.kh; a.kw = d.kw; a.sh = d.sh; a.sw = d.sw; a.pt = d.pt; a.pl = d.pl;
  a.dh = d.dh; a.dw = d.dw; a.ins_h = d.ins_h; a.ins_w = d.ins_w;
  a.c16 = w->c16; a.k16 = w->k16; a.kp = w->kp;
  a.npix = d.n * d.oh * d.ow;
#ifdef TPUHIP_TRACE
  a.trace = getenv("TPUHIP_TRACE_PTR") ? (unsigned long long *)strtoull(getenv("TPUHIP_TRACE_PTR"), nullptr, 16) : nullptr;
#endif
  a.linear = d.kh == 1 && d.kw == 1 && d.sh == 1 && d.sw == 1 && d.pt == 0 && d.pl == 0 && d.pb == 0 &&
             d.pr == 0 && d.ih == d.oh && d.iw == d.ow && d.ins_h == 0 && d.ins_w == 0;
  a.lo = (d.do_relu && !d.relu_first) ? 0 : -128;
  a.relu_first = (d.do_relu && d.relu_first) ? 1 : 0;
  a.store_y = 1;
  a.magic_kw = (1u << 20) / (uint32_t)d.kw + 1;
  a.x_bytes = (uint32_t)((int64_t)d.n * d.ih * d.iw * d.x_cs);
  a.split_oc = w->split_oc;
  a.y2_cs = w->y2_cs;
  a.lo2 = w->relu2 ? 0 : -128;
  a.stem_pw = 127 * d.sw + 8;
  a.magic_pw = (1u << 20) / (uint32_t)a.stem_pw + 1;
  if (w->algo == ALGO_MFMA) {
    const TileCfg &t = kTiles[w->tile];
    a.magic_c16 = (1u << 20) / (uint32_t)w->c16 + 1;
    a.w_bytes = (uint32_t)((int64_t)w->ocp * w->kp);
    a.magic_ow = d.ow > 1 ? (uint32_t)(((1ull << 32) + d.ow - 1) / (uint64_t)d.ow) : 0;
    a.magic_oh = d.oh > 1 ? (uint32_t)(((1ull << 32) + d.oh - 1) / (uint64_t)d.oh) : 0;
    a.n_oc_tiles = w->ocp / t.bm;
    a.n_tiles = (int)(ceil_div64(a.npix, t.bn) * a.n_oc_tiles);
    a.magic_oc_tiles = 0;   // set below, once the tile count is final
    // workgroups per XCD (a workgroup of the LDS-free kernel holds four wave tiles)
    const int n_wgs = t.reg == 1 ? (a.n_tiles + 3) / 4 : a.n_tiles;
    a.tiles_per_xcd = (n_wgs + 7) / 8;
    a.wgs_per_xcd = a.tiles_per_xcd;
    if (t.reg == 4 || t.reg == 6) {
      const int th = t.reg == 4 ? patch_rows(d, t) : patch2_rows(d, t);
      const int tiles_per_img = (d.oh + th - 1) / th;
      const int n_pix_tiles = d.n * tiles_per_img;
      a.n_tiles = n_pix_tiles * a.n_oc_tiles;
      a.tiles_per_xcd = (n_pix_tiles + 7) / 8 * a.n_oc_tiles;
      a.wgs_per_xcd = a.tiles_per_xcd;
      a.stem_pw = d.ow + 2;
      a.magic_pw = (1u << 20) / (uint32_t)a.stem_pw + 1;
      a.pstep_pix = th;
      a.pstep_n = tiles_per_img;
      a.pstep_oh = w->c16 == 4 ? 2 : w->c16 == 8 ? 3 : w->c16 == 16 ? 4 : 5;     // log2(C / 16)
      a.pstep_ow = w->c16 == 4 ? 2 : w->c16 == 8 ? 1 : 0;                        // swizzle shift
      if (t.reg == 6) {
        int lgc = 6;
        while ((1 << lgc) < d.ic) ++lgc;
        a.pstep_oh = lgc;                                                        // log2(C)
        const uint32_t rowchunks = (uint32_t)a.stem_pw * (uint32_t)(d.ic / 16);
        a.magic_c16 = (uint32_t)(((1ull << 32) + rowchunks - 1) / rowchunks);    // q / rowchunks == umulhi(q, magic), q < 2^16
        a.pstep_ow = (int)patch2_lds_bytes(t, th, d.ow, d.ic);                   // dynamic LDS of the launch
      }
    }
    if (t.reg == 7) {
      const Patch3Plan pl = patch3_plan(d, t);
      const int tiles_per_img = (d.oh + pl.th - 1) / pl.th;
      const int n_pix_tiles = pl.imgs > 1 ? (d.n + pl.imgs - 1) / pl.imgs : d.n * tiles_per_img;
      a.n_tiles = n_pix_tiles * a.n_oc_tiles;
      a.tiles_per_xcd = (n_pix_tiles + 7) / 8 * a.n_oc_tiles;
      a.wgs_per_xcd = a.tiles_per_xcd;
      a.stem_pw = d.ow + 2;
      a.pstep_pix = pl.th;
      a.pstep_n = tiles_per_img;
      a.tile_imgs = pl.imgs;
      int lgc = 6;
      while ((1 << lgc) < d.ic) ++lgc;
      a.pstep_oh = lgc;                                                          // log2(C)
      const uint32_t rowchunks = (uint32_t)d.iw * (uint32_t)(d.ic / 16);
      a.magic_c16 = (uint32_t)(((1ull << 32) + rowchunks - 1) / rowchunks);      // q / rowchunks == umulhi(q, magic), q < 2^16
      a.magic_kw = (uint32_t)(((1ull << 32) + (uint64_t)d.oh - 1) / (uint64_t)d.oh);   // span row / H
      a.magic_oh = (uint32_t)(((1ull << 32) + (uint64_t)(d.oh * d.ow) - 1) / (uint64_t)(d.oh * d.ow));
      a.pstep_ow = (int)pl.lds;                                                  // dynamic LDS of the launch
    }
    if (t.reg == 3 || t.reg == 5) {
      // every XCD owns a run of whole pixel tiles; a workgroup keeps its channel tile
      const int n_pix_tiles = a.n_tiles / a.n_oc_tiles;
      a.tiles_per_xcd = (n_pix_tiles + 7) / 8 * a.n_oc_tiles;
      const int slots = std::max(1, ctx->num_cu / 8) * persist_wgs_per_cu(w);
      a.wgs_per_xcd = std::min(a.tiles_per_xcd, std::max(1, slots / a.n_oc_tiles) * a.n_oc_tiles);
      a.pstep_pix = a.wgs_per_xcd / a.n_oc_tiles * t.bn;
      a.pstep_ow = a.pstep_pix % d.ow;
      a.pstep_oh = a.pstep_pix / d.ow % d.oh;
      a.pstep_n = a.pstep_pix / d.ow / d.oh;
    }
  }
  if (w->algo == ALGO_MFMA && a.n_oc_tiles > 1 &&
      ((int64_t)a.n_tiles + 8 * (int64_t)a.tiles_per_xcd) * a.n_oc_tiles < (1ll << 32))
    a.magic_oc_tiles = (uint32_t)(((1ull << 32) + a.n_oc_tiles - 1) / (uint64_t)a.n_oc_tiles);
  *out = a;
}

void launch_conv_mfma(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const ConvArgs &a) {
  dim3 grid((unsigned)(a.wgs_per_xcd * 8));
  if (kTiles[w->tile].reg == 5) {
    launch_pw(ctx, w->tile, grid, a);
    return;
  }
  if (kTiles[w->tile].reg == 6) {
    launch_patch2(ctx, w->tile, grid, a, (unsigned)a.pstep_ow);
    return;
  }
  if (kTiles[w->tile].reg == 7) {
    launch_patch3(ctx, w->tile, grid, a, (unsigned)a.pstep_ow);
    return;
  }
  const bool uni = (w->c16 % (tile_bk(kTiles[w->tile]) / 16)) == 0;
  if (w->smallc) {
    if (w->fast)
      launch_mfma<true, kModeSmallC>(ctx, w->tile, grid, a);
    else
      launch_mfma<false, kModeSmallC>(ctx, w->tile, grid, a);
  } else if (w->fast && uni) {
    launch_mfma<true, kModeUniform>(ctx, w->tile, grid, a);
  } else if (w->fast) {
    launch_mfma<true, kModeGeneral>(ctx, w->tile, grid, a);
  } else if (uni) {
    launch_mfma<false, kModeUniform>(ctx, w->tile, grid, a);
  } else {
    launch_mfma<false, kModeGeneral>(ctx, w->tile, grid, a);
  }
}

// Times every candidate tile on the layer's real buffers (the kernels are
// idempotent and bit-identical across tiles) and keeps the fastest.
// what runs behind the requantisation in the epilogue
struct PostOps {
  const int8_t *lut = nullptr;   // host table, 256 entries
  void *lut_out = nullptr;
  const tpuhip_fused_add *f = nullptr;
  const void *add_src = nullptr;
  void *add_out = nullptr;
  void *y2 = nullptr;            // second result of a packed pair
  const tpuhip_pool_desc *pool = nullptr;   // a 3x3 / stride 2 max pool behind the stem
  void *pool_out = nullptr;
  bool has_add() const { return f && f->enable; }
  bool any() const { return lut || has_add() || y2 || pool; }
};

// The stem + max pool launch: whether it applies, and its tiling.  rows = pooled rows per
// workgroup: as many as LDS holds (patch + conv tile), fewer while the launch would leave
// compute units without a tile, then evened out over the image.
bool stem_pool_plan(const tpuhip_conv_weights *w, const tpuhip_pool_desc &p, int num_cu, StemPoolArgs *out,
                    unsigned *lds_bytes) {
  const tpuhip_conv_desc &d = w->d;
  if (w->algo != ALGO_STEM || !w->fast || !d.do_relu || d.relu_first) return false;
  if (d.oc <= 32 || d.oc > 64 || d.kh < 4 || d.kh > 7 || d.kw > 8 || d.sw > 2 || d.ow < 2) return false;
  if (p.kh != 3 || p.kw != 3 || p.sh != 2 || p.sw != 2 || p.pt < 0 || p.pt > 1 || p.pl < 0 || p.pl > 1) return false;
  if (p.n != d.n || p.c != d.oc || p.ih != d.oh || p.iw != d.ow || p.x_cs != d.y_cs) return false;
  if (p.oh < 1 || p.ow < 1 || p.y_cs < round_up(d.oc, 16) || p.y_cs % 8) return false;
  // every window holds at least one conv pixel
  if (2 * (p.oh - 1) - p.pt > d.oh - 1 || 2 * (p.ow - 1) - p.pl > d.ow - 1) return false;
  const int pw = round_up((d.ow - 1) * d.sw + 8, 4);
  auto bytes_crows = [&](int crows) { return stem_pool_lds_bytes((crows - 1) * d.sh + d.kh, pw, crows * d.ow); };
  auto fits_crows = [&](int crows) {
    return bytes_crows(crows) <= 160u * 1024 && crows * d.ow < 65536 &&
           ((crows - 1) * d.sh + d.kh) * pw <= kStemPoolLoads * 512;
  };
  auto fits = [&](int rows) { return fits_crows(2 * rows + 1); };
  if (!fits(1)) return false;
  int rows = 1;
  while (rows < p.oh && fits(rows + 1)) ++rows;
  while (rows > 1 && (int64_t)d.n * ((p.oh + rows - 1) / rows) < num_cu) --rows;
  const int per_image = (p.oh + rows - 1) / rows;
  rows = (p.oh + per_image - 1) / per_image;
  StemPoolArgs s{};
  s.poh = p.oh; s.pow = p.ow; s.ppt = p.pt; s.ppl = p.pl; s.p_cs = p.y_cs;
  s.rows = rows;
  s.tiles_per_image = per_image;
  s.n_tiles = d.n * per_image;
  s.crows = 2 * rows + 1;
  s.crows_last = std::max(2 * (p.oh - (per_image - 1) * rows) + 1, d.oh - (2 * (per_image - 1) * rows - p.pt));
  if (!fits_crows(std::max(s.crows, s.crows_last))) return false;
  s.prows = (std::max(s.crows, s.crows_last) - 1) * d.sh + d.kh;
  s.pw = pw;
  s.magic_pw = (uint32_t)(((1ull << 32) + pw - 1) / (uint64_t)pw);
  s.magic_pow = p.ow > 1 ? (uint32_t)(((1ull << 32) + p.ow - 1) / (uint64_t)p.ow) : 0;
  if (p.ow == 1) return false;
  *out = s;
  *lds_bytes = bytes_crows(std::max(s.crows, s.crows_last));
  return true;
}

void apply_fusion(ConvArgs *a, const void *y, const PostOps &p) {
  if (p.lut) {
    a->has_lut = 1;
    a->lut_dst = (int8_t *)p.lut_out;
    memcpy(a->lut.w, p.lut, 256);
  }
  if (p.has_add()) {
    a->add_src = (const int8_t *)p.add_src;
    a->add_dst = (int8_t *)p.add_out;
    a->add_m_src = p.f->m_src;
    a->add_m_conv = p.f->m_conv;
    a->add_rshift = p.f->rshift;
    a->add_relu = p.f->do_relu ? 1 : 0;
    a->add_pk = std::abs(p.f->m_src) <= 127 && std::abs(p.f->m_conv) <= 127 && p.f->rshift <= 8;
  }
  a->store_y = y != nullptr;
  a->y2 = (int8_t *)p.y2;
}

// The fused add (if any) is part of what is timed: it shifts the balance between
// the tile shapes.  Every launch recomputes the same bytes, so repeating it is safe
// as long as the sum is not written over its own input.
int autotune_mfma(tpuhip_ctx *ctx, tpuhip_conv_weights *w, const void *x, void *y,
                  const PostOps &post) {
  hipEvent_t e0, e1;
  TPUHIP_CHECK_HIP(hipEventCreate(&e0));
  TPUHIP_CHECK_HIP(hipEventCreate(&e1));
  float best_ms = 1e30f;
  int best = -1;
  int rc = TPUHIP_OK;
  for (int t = 0; t < kNumTiles && !rc; ++t) {
    if (!tile_is_candidate(w->d, t)) continue;
    if (post.lut && !tile_has_lds_epilogue(t)) continue;
    if (w->split_oc && kTiles[t].reg == 4) continue;   // the patch kernel writes one result
    if (kTiles[t].reg == 5 && (!w->fast || w->split_oc % kTiles[t].bm)) continue;
    if ((kTiles[t].reg == 6 || kTiles[t].reg == 7) && (!w->fast || w->split_oc)) continue;
    rc = pack_mfma_weights(ctx, w, t);
    if (rc) break;
    ConvArgs a;
    fill_args(ctx, w, x, y, &a);
    apply_fusion(&a, y, post);
    for (int i = 0; i < 2; ++i) launch_conv_mfma(ctx, w, a);
    hipError_t er = hipEventRecord(e0, ctx->stream);
    for (int i = 0; i < 5; ++i) launch_conv_mfma(ctx, w, a);
    if (er == hipSuccess) er = hipEventRecord(e1, ctx->stream);
    hipError_t es = hipEventSynchronize(e1);
    const hipError_t el = hipGetLastError();
    if (es == hipSuccess) es = er;
    if (es != hipSuccess || el != hipSuccess) {
      // a variant that cannot be launched is skipped; the layer fails only if none can
      set_error(TPUHIP_ERR_HIP, "conv autotune: tile %s failed: %s", kTiles[t].name,
                hipGetErrorString(es != hipSuccess ? es : el));
      if (getenv("TPUHIP_DEBUG")) fprintf(stderr, "%s\n", tpuhip_last_error());
      continue;
    }
    float ms = 0;
    if (hipEventElapsedTime(&ms, e0, e1) != hipSuccess) continue;
    if (ms < best_ms) {
      best_ms = ms;
      best = t;
    }
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc) return rc;
  if (best < 0) return TPUHIP_ERR_HIP;   // the last launch error is still the message
  if (best != w->tile) rc = pack_mfma_weights(ctx, w, best);
  w->tuned = true;
  w->host_filter.clear();
  w->host_filter.shrink_to_fit();
  return rc;
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

  const int icg = d.ic / d.g;
  const bool dense = d.g == 1 && d.ins_h == 0 && d.ins_w == 0;
  const bool depthwise = d.g == d.ic && d.g == d.oc && d.ins_h == 0 && d.ins_w == 0;
  int algo = d.algo, forced_tile = -1;
  if (algo >= 16) {   // MFMA with an explicit tile variant (tests, tuning)
    forced_tile = algo - 16;
    algo = ALGO_MFMA;
    TPUHIP_REQUIRE(forced_tile < kNumTiles, "conv: unknown MFMA tile %d", forced_tile);
  }
  // the stem kernel: one dword per pixel, the taps of a filter row side by side
  const bool stem_ok = dense && d.ic <= 4 && d.dh == 1 && d.dw == 1 && d.kw <= 8 && d.kh <= 7 &&
                       d.sw <= 2 && d.oc <= 64;
  if (algo == ALGO_AUTO)
    algo = stem_ok ? ALGO_STEM : dense ? ALGO_MFMA : depthwise ? ALGO_DEPTHWISE : ALGO_DIRECT;
  TPUHIP_REQUIRE(algo >= ALGO_DIRECT && algo <= ALGO_STEM, "conv: unknown algo %d", d.algo);
  TPUHIP_REQUIRE(algo != ALGO_STEM || stem_ok,
                 "conv: the stem path needs g == 1, ic <= 4, oc <= 64, kh <= 7, kw <= 8, stride_w <= 2, "
                 "no dilation, no inserted zeros");
  TPUHIP_REQUIRE(d.x_cs % 16 == 0 || algo == ALGO_STEM,
                 "conv: only the stem path (g == 1, ic <= 4, oc <= 64, kh <= 7, kw <= 8, stride_w <= 2) reads an input "
                 "with a 4-byte channel stride");
  // the MFMA kernel locates a K group with multiply-shift divisions that are exact
  // for at most 4094 groups of at most 256 16-channel groups each
  const bool mfma_ok = dense && round_up(d.ic, 16) / 16 <= 256 &&
                       (int64_t)d.kh * d.kw * (round_up(d.ic, 16) / 16) + 128 < 4095 &&
                       (int64_t)round_up(d.oc, 128) * (d.kh * d.kw * round_up(d.ic, 16) + 256) <
                           (1ll << 31);
  if (d.algo == ALGO_AUTO && algo == ALGO_MFMA && !mfma_ok) algo = ALGO_DIRECT;
  // a matrix product packed fragment by fragment (tpuhip_fc_prepack): the FullyConnected kernels
  // take any K whose packed filter stays within a buffer descriptor's 2 GiB
  const bool fc_form = dense && forced_tile >= 0 && std::string(kTiles[forced_tile].name) == "mfma_reg_32x32" &&
                       d.relu_first && d.ih == 1 && d.iw == 1 && d.kh == 1 && d.kw == 1 &&
                       (int64_t)round_up(d.oc, 32) * round_up(d.ic, 64) < (1ll << 31);
  TPUHIP_REQUIRE(algo != ALGO_MFMA || mfma_ok || fc_form,
                 "conv: MFMA path needs g == 1, no inserted zeros, ic <= 4096 and K < 65000");
  TPUHIP_REQUIRE((algo != ALGO_DEPTHWISE && algo != ALGO_DEPTHWISE_DOT) || depthwise,
                 "conv: depthwise path needs g == ic == oc and no inserted zeros");

  auto *cw = new tpuhip_conv_weights();
  cw->d = d;
  cw->algo = algo;
  cw->fc_only = algo == ALGO_MFMA && !mfma_ok;
  std::vector<int8_t> packed;
  const size_t per_oc = (size_t)icg * d.kh * d.kw;
  if (algo == ALGO_MFMA) {
    cw->c16 = round_up(d.ic, 16) / 16;
    cw->k16 = d.kh * d.kw * cw->c16;   // refined per tile in pack_mfma_weights
    cw->host_filter.assign(filter, filter + (size_t)d.oc * per_oc);
    const int tile = forced_tile >= 0 ? forced_tile : pick_tile(d, cw->k16, ctx->num_cu);
    if (int rc = pack_mfma_weights(ctx, cw, tile)) {
      tpuhip_conv2d_weights_destroy(ctx, cw);
      return rc;
    }
    cw->tuned = forced_tile >= 0 || !ctx->autotune;
    if (cw->tuned) {
      cw->host_filter.clear();
      cw->host_filter.shrink_to_fit();
    }
  } else if (algo == ALGO_DEPTHWISE) {
    // diagonal MFMA A fragments: [32-channel block][tap][lane][16 bytes]; lane l holds row
    // l & 31 (channel mfma_row_to_oc(row) of the block), K bytes 16*(l >> 5) .. +15
    cw->ocp = round_up(d.oc, 16);
    const int taps = d.kh * d.kw, n_cb = (cw->ocp + 31) / 32;
    packed.assign((size_t)n_cb * taps * 1024, 0);
    for (int cb = 0; cb < n_cb; ++cb)
      for (int t = 0; t < taps; ++t)
        for (int lane = 0; lane < 64; ++lane) {
          const int ch_in_block = mfma_row_to_oc(lane & 31, 1);
          const int ch = cb * 32 + ch_in_block;
          const int j = ch_in_block - 16 * (lane >> 5);
          if (ch < d.oc && j >= 0 && j < 16)
            packed[((size_t)(cb * taps + t) * 64 + lane) * 16 + j] = filter[(size_t)ch * taps + t];
        }
  } else if (algo == ALGO_STEM) {
    // A fragments [32-channel block][filter row][lane][16 bytes]: lane l holds MFMA row l & 31
    // (channel mfma_row_to_oc(row) of the block) and K bytes 16*(l >> 5) .. +15 of the
    // 32-byte filter row, K byte = 4 * kw + channel
    cw->ocp = round_up(d.oc, 16);
    const int tm = d.oc <= 32 ? 1 : 2, khp = d.kh <= 3 ? 3 : 7;
    packed.assign((size_t)tm * khp * 1024, 0);
    for (int i = 0; i < tm; ++i)
      for (int r = 0; r < d.kh; ++r)
        for (int lane = 0; lane < 64; ++lane) {
          const int oc = i * 32 + mfma_row_to_oc(lane & 31, 1);
          if (oc >= d.oc) continue;
          for (int j = 0; j < 16; ++j) {
            const int kw = (lane >> 5) * 4 + j / 4, c = j % 4;
            if (kw < d.kw && c < d.ic)
              packed[((size_t)(i * khp + r) * 64 + lane) * 16 + j] =
                  filter[(((size_t)oc * d.ic + c) * d.kh + r) * d.kw + kw];
          }
        }
  } else if (algo == ALGO_DEPTHWISE_DOT) {
    // [tap group][channel][4 taps]: one dword per channel and group of four taps
    cw->ocp = round_up(d.oc, 16);
    const int groups = std::max(3, (d.kh * d.kw + 3) / 4);   // the kernel holds three groups in registers
    packed.assign((size_t)groups * cw->ocp * 4, 0);
    for (int c = 0; c < d.oc; ++c)
      for (int tap = 0; tap < d.kh * d.kw; ++tap)
        packed[((size_t)(tap / 4) * cw->ocp + c) * 4 + tap % 4] = filter[(size_t)c * d.kh * d.kw + tap];
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
  // epilogue parameters, indexed by the true output channel.  `fast` holds when,
  // for every channel, 1 <= rshift and |acc + bias| + 1 + 2^(rshift-1) cannot reach
  // 2^31: |acc| <= 128 * sum|w|, and |x| <= |v| + 1 after the doubling high multiply.
  const size_t nparam = (size_t)round_up(d.oc, 256) + 16;   // covers every tile's padding
  std::vector<int32_t> b32(nparam, 0);
  std::vector<QParam> qp(nparam);
  bool fast = true;
  for (int i = 0; i < (int)qp.size(); ++i) {
    QParam q{};
    if (i < d.oc) {
      b32[i] = (d.with_bias && bias) ? bias[i] : 0;
      q.mult = multiplier[i];
      q.rshift = rshift[i];
      q.mask = (int32_t)((1ll << rshift[i]) - 1);
      q.hpot = rshift[i] > 0 ? (int32_t)(1ll << (rshift[i] - 1)) : 0;
      int64_t sumw = 0;
      for (size_t k = 0; k < per_oc; ++k) sumw += std::abs((int)filter[(size_t)i * per_oc + k]);
      const int64_t bound = 128 * sumw + std::llabs((long long)b32[i]) + 1 + q.hpot;
      if (rshift[i] < 1 || bound >= (1ll << 31)) fast = false;
    } else {
      q.rshift = 1;   // pad channels: multiplier 0 gives 0 on either path
      q.mask = 1;
      q.hpot = 1;
    }
    qp[i] = q;
  }
  cw->fast = fast ? 1 : 0;
  int rc = TPUHIP_OK;
  if (algo != ALGO_MFMA) {
    rc = tpuhip_malloc(ctx, packed.size(), (void **)&cw->w);
    if (!rc) rc = tpuhip_upload(ctx, cw->w, packed.data(), packed.size());
  }
  if (!rc) rc = tpuhip_malloc(ctx, b32.size() * sizeof(int32_t), (void **)&cw->bias);
  if (!rc) rc = tpuhip_malloc(ctx, qp.size() * sizeof(QParam), (void **)&cw->qp);
  if (!rc) rc = tpuhip_upload(ctx, cw->bias, b32.data(), b32.size() * sizeof(int32_t));
  if (!rc) rc = tpuhip_upload(ctx, cw->qp, qp.data(), qp.size() * sizeof(QParam));
  if (!rc && algo != ALGO_DIRECT) {
    std::vector<int32_t> planes(3 * nparam);
    for (size_t i = 0; i < nparam; ++i) {
      planes[i] = qp[i].mult;
      planes[nparam + i] = qp[i].rshift;
      planes[2 * nparam + i] = qp[i].hpot;
    }
    cw->nparam = (int)nparam;
    rc = tpuhip_malloc(ctx, planes.size() * sizeof(int32_t), (void **)&cw->qplanes);
    if (!rc) rc = tpuhip_upload(ctx, cw->qplanes, planes.data(), planes.size() * sizeof(int32_t));
    // (acc + bias) * mult + 2^30 == acc * mult + c: the addend of the requantisation's 64-bit
    // multiply-add, as a plane of low and a plane of high words
    std::vector<int32_t> c64(4 * nparam);
    for (size_t i = 0; i < nparam; ++i) {
      const int64_t c = (int64_t)b32[i] * (int64_t)qp[i].mult + (1ll << 30);
      const int64_t cr = c + ((int64_t)qp[i].hpot << 31);
      c64[2 * i] = (int32_t)(uint32_t)(c & 0xffffffffll);
      c64[2 * i + 1] = (int32_t)(c >> 32);
      c64[2 * nparam + 2 * i] = (int32_t)(uint32_t)(cr & 0xffffffffll);
      c64[2 * nparam + 2 * i + 1] = (int32_t)(cr >> 32);
    }
    if (!rc) rc = tpuhip_malloc(ctx, c64.size() * sizeof(int32_t), (void **)&cw->qc64);
    if (!rc) rc = tpuhip_upload(ctx, cw->qc64, c64.data(), c64.size() * sizeof(int32_t));
  }
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
  int rc2 = tpuhip_free(ctx, w->bias);
  int rc3 = tpuhip_free(ctx, w->qp);
  int rc4 = tpuhip_free(ctx, w->qplanes);
  int rc5 = tpuhip_free(ctx, w->qc64);
  delete w;
  return rc ? rc : rc2 ? rc2 : rc3 ? rc3 : rc4 ? rc4 : rc5;
}

const char *tpuhip_conv2d_tile_name(int tile) {
  return tile >= 0 && tile < kNumTiles ? kTiles[tile].name : nullptr;
}

int tpuhip_conv2d_can_fuse_table(const tpuhip_conv_weights *w) {
  if (!w) return 0;
  if (w->algo == ALGO_DEPTHWISE || w->algo == ALGO_DEPTHWISE_DOT || w->algo == ALGO_STEM) return 1;
  return w->algo == ALGO_MFMA && (!w->tuned || tile_has_lds_epilogue(w->tile)) ? 1 : 0;
}

int tpuhip_conv2d_set_input_stride(tpuhip_conv_weights *w, int x_cs) {
  TPUHIP_REQUIRE(w, "tpuhip_conv2d_set_input_stride: NULL argument");
  TPUHIP_REQUIRE(x_cs >= w->d.ic && (x_cs % 16 == 0 || x_cs == 4), "conv: input channel stride %d must be 4 or a multiple of 16 covering %d channels", x_cs, w->d.ic);
  if (x_cs == 4 && (w->algo != ALGO_STEM || w->split_oc))
    return set_error(TPUHIP_ERR_UNSUPPORTED, "conv: only the stem path reads an input with a 4-byte channel stride");
  TPUHIP_REQUIRE((int64_t)w->d.n * (w->d.ih + w->d.pt + w->d.pb + 2) * (w->d.iw + w->d.pl + w->d.pr + 2) * x_cs < (1ll << 31),
                 "conv: tensor too large");
  w->d.x_cs = x_cs;
  return TPUHIP_OK;
}

const char *tpuhip_conv2d_algo_name(const tpuhip_conv_weights *w) {
  if (!w) return "null";
  switch (w->algo) {
    case ALGO_DIRECT: return "direct";
    case ALGO_DEPTHWISE: return "depthwise";
    case ALGO_DEPTHWISE_DOT: return "depthwise_dot";
    case ALGO_STEM: return "stem";
    case ALGO_MFMA: return kTiles[w->tile].name;
  }
  return "?";
}

static int run_fc_one(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y);

// Whether the row-segment depthwise kernel takes the layer, and its blocks: R row segments of
// W lanes per wave, chosen for the fewest blocks per image.
static bool dw_rows_plan(const tpuhip_conv_weights *w, const ConvArgs &a, DwRowsArgs *out) {
  const tpuhip_conv_desc &d = w->d;
  if (w->algo != ALGO_DEPTHWISE || !w->fast || d.relu_first || d.kh > 3 || d.kw > 3 || a.add_dst) return false;
  // input rows and the row pitch fit the 24-bit multiply of the address arithmetic
  if (d.ih >= (1 << 22) || (int64_t)d.iw * d.x_cs >= (1ll << 23) || (int64_t)d.ih * d.iw * d.x_cs >= (1ll << 31)) return false;
  const int halo = (d.kw == 3 && d.sw == 1 && d.dw == 1) ? 1 : 0;
  int64_t best = -1;
  for (int rows = 1; rows <= 4; ++rows) {
    const int width = 32 / rows, valid = width - 2 * halo;
    if (valid < 1) continue;
    const int64_t blocks = (int64_t)((d.oh + rows - 1) / rows) * ((d.ow + valid - 1) / valid);
    if (best < 0 || blocks < best) {
      best = blocks;
      out->rows = rows; out->width = width; out->valid = valid; out->halo = halo;
      out->rblocks = (d.oh + rows - 1) / rows;
      out->xblocks = (d.ow + valid - 1) / valid;
    }
  }
  if (best < 0 || best * d.n >= (1ll << 30) || out->rblocks >= (1 << 15) || out->xblocks >= (1 << 15)) return false;
  out->nblocks = (int)(best * d.n);
  auto magic = [](int dv) { return dv > 1 ? (uint32_t)(((1ull << 32) + dv - 1) / (uint64_t)dv) : 0u; };
  out->magic_x = magic(out->xblocks);
  out->magic_r = magic(out->rblocks);
  out->magic_w = magic(out->width);
  return true;
}

// the walk of the row-segment depthwise kernel for a launch of `wgs` workgroups (a multiple of 8)
static void dw_rows_walk(DwRowsArgs *r, unsigned wgs, int n_cb) {
  r->nslots = std::max(1, std::min((int)(wgs / 8) * 4 / n_cb, 1 << 15));
  r->d_xb = r->nslots % r->xblocks;
  r->d_rb = (r->nslots / r->xblocks) % r->rblocks;
  r->d_n = r->nslots / (r->xblocks * r->rblocks);
  const int per_xcd = (r->nblocks + 7) / 8;
  for (int x = 0; x < 8; ++x) {
    const int64_t b = (int64_t)x * per_xcd;
    r->start_xb[x] = (int)(b % r->xblocks);
    r->start_rb[x] = (int)((b / r->xblocks) % r->rblocks);
    r->start_n[x] = (int)(b / ((int64_t)r->xblocks * r->rblocks));
  }
}

static int run_conv(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
                    const PostOps &post) {
  if (w->fc_only) {
    TPUHIP_REQUIRE(!post.any() && y, "conv: a FullyConnected of more than 4096 input channels takes no fused work");
    return run_fc_one(ctx, w, x, y);
  }
  if (w->algo == ALGO_MFMA && !w->tuned) {
    // first use: pick the tile by measurement (not capturable into a HIP graph).  The
    // fused work is timed with it unless the sum would overwrite its own operand.
    PostOps tp = post;
    if (tp.has_add() && tp.add_out == tp.add_src) tp.f = nullptr;
    void *ty = y;
    if (!ty && !tp.has_add() && !(tp.lut && tp.lut_out)) {
      // tuning writes the plain conv result somewhere: borrow a buffer
      const size_t bytes = (size_t)w->d.n * w->d.oh * w->d.ow * w->d.y_cs;
      if (int rc = tpuhip_malloc(ctx, bytes, &ty)) return rc;
    }
    int rc = autotune_mfma(ctx, const_cast<tpuhip_conv_weights *>(w), x, ty, tp);
    if (ty != y) tpuhip_free(ctx, ty);
    if (rc) return rc;
  }
  TPUHIP_REQUIRE(!post.lut || w->algo == ALGO_DEPTHWISE || w->algo == ALGO_DEPTHWISE_DOT ||
                     w->algo == ALGO_STEM ||
                     (w->algo == ALGO_MFMA && tile_has_lds_epilogue(w->tile)),
                 "conv: kernel variant %s cannot fuse a table", tpuhip_conv2d_algo_name(w));
  TPUHIP_REQUIRE(!(w->algo == ALGO_MFMA && kTiles[w->tile].reg == 4) || (!w->split_oc && patch_rows(w->d, kTiles[w->tile]) > 0),
                 "conv: tile variant %s needs a single 3x3 / stride 1 / pad 1 conv with 64, 128, 256 or 512 input "
                 "channels on a map narrow enough for its row patch", kTiles[w->tile].name);
  TPUHIP_REQUIRE(!(w->algo == ALGO_MFMA && kTiles[w->tile].reg == 5) ||
                     (pw_shape_ok(w->d, kTiles[w->tile]) && w->fast && w->split_oc % kTiles[w->tile].bm == 0),
                 "conv: tile variant %s needs an unpadded 1x1 conv with 5 to %d input channels, right shifts of at "
                 "least 1 and sums that cannot overflow the rounding, and a pair split at a tile boundary",
                 kTiles[w->tile].name, kTiles[w->tile].bk);
  TPUHIP_REQUIRE(!(w->algo == ALGO_MFMA && kTiles[w->tile].reg == 7) ||
                     (!w->split_oc && w->fast && patch3_plan(w->d, kTiles[w->tile]).th > 0),
                 "conv: tile variant %s needs a single 3x3 / stride 1 / pad 1 conv with 64, 128, 256, 512 or 1024 input "
                 "channels on a map narrow enough for its row patch, right shifts of at least 1 and sums that cannot "
                 "overflow the rounding", kTiles[w->tile].name);
  TPUHIP_REQUIRE(!(w->algo == ALGO_MFMA && kTiles[w->tile].reg == 6) ||
                     (!w->split_oc && w->fast && patch2_rows(w->d, kTiles[w->tile]) > 0),
                 "conv: tile variant %s needs a single 3x3 / stride 1 / pad 1 conv with 64, 128, 256, 512 or 1024 input "
                 "channels on a map narrow enough for its row patch, right shifts of at least 1 and sums that cannot "
                 "overflow the rounding", kTiles[w->tile].name);
  TPUHIP_REQUIRE((w->split_oc != 0) == (post.y2 != nullptr),
                 "conv: weights packed as a pair run through tpuhip_conv2d_pair_i8 (and only they do)");
  ConvArgs a;
  fill_args(ctx, w, x, y, &a);
  apply_fusion(&a, y, post);
  if (w->algo == ALGO_MFMA) {
    launch_conv_mfma(ctx, w, a);
  } else if (w->algo == ALGO_DEPTHWISE) {
    // one wave per (32-channel block, 32-pixel block); a resident set of workgroups, each
    // wave walking pixel blocks of its channel block
    const int n_cb = (a.ocw + 31) / 32, n_pb = (a.npix + 31) / 32;
    DwRowsArgs dr;
    if (dw_rows_plan(w, a, &dr)) {
      // the row-segment form: up to 3 x 3 taps, the layer's overflow-free requantisation, no fused add
      const int64_t waves_r = (int64_t)n_cb * dr.nblocks;
      const unsigned wgs = 8 * (unsigned)std::max<int64_t>(
          (n_cb + 3) / 4, std::min<int64_t>(ceil_div64(waves_r, 32), std::max(1, ctx->num_cu * (dr.halo ? 4 : 3) / 8)));
      const bool shift = dr.halo == 1;
      dw_rows_walk(&dr, wgs, n_cb);
      a.magic_c16 = n_cb > 1 ? (uint32_t)(((1ull << 32) + n_cb - 1) / (uint64_t)n_cb) : 0u;   // wave index / n_cb
      auto kernel = shift ? conv_depthwise_rows_kernel<true> : conv_depthwise_rows_kernel<false>;
      if (ctx->prof_start)
        hipExtLaunchKernelGGL(kernel, dim3(wgs), dim3(256), 0, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a, dr);
      else
        hipLaunchKernelGGL(kernel, dim3(wgs), dim3(256), 0, ctx->stream, a, dr);
      TPUHIP_CHECK_HIP(hipGetLastError());
      return TPUHIP_OK;
    }
    const int64_t waves = (int64_t)n_cb * n_pb;
    // a multiple of 8 workgroups, every XCD's share holding at least one wave per channel block
    const unsigned blocks = 8 * (unsigned)std::max<int64_t>(
        (n_cb + 3) / 4, std::min<int64_t>(ceil_div64(waves, 32), std::max(1, ctx->num_cu * 3 / 8)));
    const dim3 grid(blocks), block(256);
    const bool regw = a.kh * a.kw <= 9;
    if (w->fast) {
      if (regw) launch(ctx, (conv_depthwise_mfma_kernel<true, true>), grid, block, a);
      else launch(ctx, (conv_depthwise_mfma_kernel<true, false>), grid, block, a);
    } else {
      if (regw) launch(ctx, (conv_depthwise_mfma_kernel<false, true>), grid, block, a);
      else launch(ctx, (conv_depthwise_mfma_kernel<false, false>), grid, block, a);
    }
  } else if (w->algo == ALGO_STEM && post.pool) {
    StemPoolArgs sp;
    unsigned lds = 0;
    TPUHIP_REQUIRE(!post.lut && !post.has_add() && post.pool_out && stem_pool_plan(w, *post.pool, ctx->num_cu, &sp, &lds),
                   "conv: this stem cannot take the max pool into its launch (tpuhip_conv2d_can_fuse_pool)");
    sp.py = (int8_t *)post.pool_out;
    a.magic_ow = (uint32_t)(((1ull << 32) + a.ow - 1) / (uint64_t)a.ow);
    TPUHIP_REQUIRE(pw_prepare(conv_stem_pool_kernel, 160u * 1024), "conv: raising the stem + pool kernel's LDS limit failed");
    const int per_cu = std::max(1, std::min(4, (int)(160u * 1024 / lds)));
    const dim3 grid((unsigned)std::min<int64_t>(sp.n_tiles, (int64_t)ctx->num_cu * per_cu)), block(512);
    if (ctx->prof_start)
      hipExtLaunchKernelGGL(conv_stem_pool_kernel, grid, block, lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a, sp);
    else
      hipLaunchKernelGGL(conv_stem_pool_kernel, grid, block, lds, ctx->stream, a, sp);
  } else if (w->algo == ALGO_STEM) {
    // one workgroup per resident slot (3 per CU), each walking (image, output row, 128-pixel
    // segment) tiles
    const int64_t tiles = (int64_t)a.n * a.oh * ((a.ow + 127) / 128);
    const bool k3 = a.kh <= 3, one = a.oc <= 32;
    const int64_t per_xcd = (tiles + 7) / 8;
    const dim3 grid((unsigned)(8 * std::min<int64_t>(per_xcd, std::max(1, ctx->num_cu * 3 / 8)))), block(256);
#define STEM(KH, TM)                                                                   \
  do {                                                                                 \
    if (w->fast) launch(ctx, (conv_stem_kernel<KH, TM, true>), grid, block, a);        \
    else launch(ctx, (conv_stem_kernel<KH, TM, false>), grid, block, a);               \
  } while (0)
    if (k3 && one) STEM(3, 1);
    else if (k3) STEM(3, 2);
    else if (one) STEM(7, 1);
    else STEM(7, 2);
#undef STEM
  } else if (w->algo == ALGO_DEPTHWISE_DOT) {
    // as many workgroups as are resident at once (3 per CU at this register count): every
    // lane then walks pixels and its filter / parameter loads are paid once (measured best)
    const int64_t total = (int64_t)a.npix * (a.ocw / 16);
    const unsigned blocks =
        (unsigned)std::max<int64_t>(1, std::min<int64_t>(ceil_div64(total, 256), (int64_t)ctx->num_cu * 3));
    const int groups = (a.kh * a.kw + 3) / 4;
    const dim3 grid(blocks), block(256);
    if (groups <= 3) {
      if (w->fast) launch(ctx, (conv_depthwise_kernel<3, true>), grid, block, a);
      else launch(ctx, (conv_depthwise_kernel<3, false>), grid, block, a);
    } else {
      if (w->fast) launch(ctx, (conv_depthwise_kernel<0, true>), grid, block, a);
      else launch(ctx, (conv_depthwise_kernel<0, false>), grid, block, a);
    }
  } else {
    const int64_t total = (int64_t)a.npix * a.ocw;
    const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(total, 256), 1 << 20);
    launch(ctx, conv_direct_kernel, dim3(blocks), dim3(256), a);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

int tpuhip_conv2d_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && w && x && y, "tpuhip_conv2d_i8: NULL argument");
  return run_conv(ctx, w, x, y, PostOps{});
}

static int check_fused_add(const tpuhip_conv_weights *w, const void *add_src, const void *add_out,
                           const tpuhip_fused_add *f) {
  TPUHIP_REQUIRE(add_src && add_out, "conv2d fused add: NULL operand");
  TPUHIP_REQUIRE(w->algo == ALGO_MFMA, "conv2d fused add: only dense convs on the MFMA path can fuse an add");
  TPUHIP_REQUIRE(f->rshift >= 0 && f->rshift <= 30, "conv2d fused add: rshift %d outside [0,30]", f->rshift);
  TPUHIP_REQUIRE(f->m_src >= -128 && f->m_src <= 127 && f->m_conv >= -128 && f->m_conv <= 127,
                 "conv2d fused add: multipliers must be int8");
  return TPUHIP_OK;
}

int tpuhip_conv2d_add_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
                         const void *add_src, void *add_out, const tpuhip_fused_add *f) {
  TPUHIP_REQUIRE(ctx && w && x && f, "tpuhip_conv2d_add_i8: NULL argument");
  TPUHIP_REQUIRE(f->enable, "conv2d_add: fusion descriptor not enabled");
  if (int rc = check_fused_add(w, add_src, add_out, f)) return rc;
  PostOps p;
  p.f = f;
  p.add_src = add_src;
  p.add_out = add_out;
  return run_conv(ctx, w, x, y, p);
}

int tpuhip_conv2d_post_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
                          const tpuhip_conv_post *post) {
  TPUHIP_REQUIRE(ctx && w && x && post, "tpuhip_conv2d_post_i8: NULL argument");
  PostOps p;
  if (post->lut) {
    TPUHIP_REQUIRE(w->algo == ALGO_MFMA || w->algo == ALGO_DEPTHWISE || w->algo == ALGO_DEPTHWISE_DOT ||
                       w->algo == ALGO_STEM,
                   "conv2d_post: only dense convs on the MFMA or stem path and depthwise convs can fuse a table");
    p.lut = post->lut;
    p.lut_out = post->lut_out;
  }
  if (post->add.enable) {
    if (int rc = check_fused_add(w, post->add_src, post->add_out, &post->add)) return rc;
    p.f = &post->add;
    p.add_src = post->add_src;
    p.add_out = post->add_out;
  }
  if (post->pool) {
    TPUHIP_REQUIRE(post->pool_out, "conv2d_post: fused pool without a result tensor");
    TPUHIP_REQUIRE(!post->lut && !post->add.enable, "conv2d_post: the fused pool takes no table and no add");
    p.pool = post->pool;
    p.pool_out = post->pool_out;
  }
  TPUHIP_REQUIRE(y || p.lut_out || p.add_out || p.pool_out, "conv2d_post: nothing would be written");
  return run_conv(ctx, w, x, y, p);
}

int tpuhip_conv2d_can_fuse_pool(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const tpuhip_pool_desc *pool) {
  if (!ctx || !w || !pool) return 0;
  StemPoolArgs sp;
  unsigned lds = 0;
  return stem_pool_plan(w, *pool, ctx->num_cu, &sp, &lds) ? 1 : 0;
}

int tpuhip_conv2d_prepack_pair(tpuhip_ctx *ctx, const tpuhip_conv_desc *da, const tpuhip_conv_desc *db,
                               const int8_t *filter_a, const int32_t *bias_a, const int32_t *mult_a,
                               const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                               const int32_t *mult_b, const int32_t *rshift_b, tpuhip_conv_weights **out) {
  TPUHIP_REQUIRE(ctx && da && db && filter_a && filter_b && mult_a && mult_b && rshift_a && rshift_b && out,
                 "tpuhip_conv2d_prepack_pair: NULL argument");
  const tpuhip_conv_desc &a = *da, &b = *db;
  if (int rc = check_desc(a)) return rc;
  if (int rc = check_desc(b)) return rc;
  TPUHIP_REQUIRE(a.n == b.n && a.ic == b.ic && a.ih == b.ih && a.iw == b.iw && a.x_cs == b.x_cs &&
                     a.oh == b.oh && a.ow == b.ow && a.kh == b.kh && a.kw == b.kw && a.sh == b.sh &&
                     a.sw == b.sw && a.pt == b.pt && a.pb == b.pb && a.pl == b.pl && a.pr == b.pr &&
                     a.dh == b.dh && a.dw == b.dw,
                 "conv pair: the two convs must read the same input through the same window geometry");
  TPUHIP_REQUIRE(a.g == 1 && b.g == 1 && !a.ins_h && !a.ins_w && !b.ins_h && !b.ins_w && !a.relu_first &&
                     !b.relu_first,
                 "conv pair: dense convs only");
  TPUHIP_REQUIRE(a.oc % 128 == 0, "conv pair: the first conv needs a multiple of 128 output channels (%d)", a.oc);
  TPUHIP_REQUIRE(a.algo == b.algo && (a.algo == ALGO_AUTO || a.algo == ALGO_MFMA || a.algo >= 16),
                 "conv pair: only the MFMA path (algo 0, 2 or 16 + tile, the same for both)");
  // one conv with the filters stacked along the output channels
  tpuhip_conv_desc m = a;
  m.oc = a.oc + b.oc;
  m.y_cs = round_up(m.oc, 16);   // only for the checks: each half keeps its own stride
  m.with_bias = (a.with_bias && bias_a) || (b.with_bias && bias_b) ? 1 : 0;
  m.algo = a.algo == ALGO_AUTO ? ALGO_MFMA : a.algo;   // the only path whose epilogue can split its output
  const size_t per_oc = (size_t)a.ic * a.kh * a.kw;
  std::vector<int8_t> filter((size_t)m.oc * per_oc);
  memcpy(filter.data(), filter_a, (size_t)a.oc * per_oc);
  memcpy(filter.data() + (size_t)a.oc * per_oc, filter_b, (size_t)b.oc * per_oc);
  std::vector<int32_t> bias((size_t)m.oc, 0), mult((size_t)m.oc), rshift((size_t)m.oc);
  for (int i = 0; i < a.oc; ++i) {
    if (a.with_bias && bias_a) bias[i] = bias_a[i];
    mult[i] = mult_a[i];
    rshift[i] = rshift_a[i];
  }
  for (int i = 0; i < b.oc; ++i) {
    if (b.with_bias && bias_b) bias[a.oc + i] = bias_b[i];
    mult[a.oc + i] = mult_b[i];
    rshift[a.oc + i] = rshift_b[i];
  }
  tpuhip_conv_weights *cw = nullptr;
  if (int rc = tpuhip_conv2d_prepack(ctx, &m, filter.data(), bias.data(), mult.data(), rshift.data(), &cw))
    return rc;
  cw->d.y_cs = a.y_cs;
  cw->split_oc = a.oc;
  cw->y2_cs = b.y_cs;
  cw->relu2 = b.do_relu ? 1 : 0;
  *out = cw;
  return TPUHIP_OK;
}

int tpuhip_conv2d_pair_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y_a, void *y_b) {
  TPUHIP_REQUIRE(ctx && w && x && y_a && y_b, "tpuhip_conv2d_pair_i8: NULL argument");
  TPUHIP_REQUIRE(w->split_oc > 0, "tpuhip_conv2d_pair_i8: weights were not packed as a pair");
  PostOps p;
  p.y2 = y_b;
  return run_conv(ctx, w, x, y_a, p);
}

// how the split-K kernel divides a packed FullyConnected: tiles, splits, K steps per split
struct FcPlan {
  int tiles, splits, steps_per_split;
  size_t bytes;   // scratch the launch needs
};

static bool fc_splitk_plan(const tpuhip_ctx *ctx, const tpuhip_conv_weights *w, FcPlan *p) {
  const tpuhip_conv_desc &d = w->d;
  // a packed FullyConnected (1x1 "image", bias before the ReLU) in the fragment order of the
  // 32x32 LDS-free tile, which is how tpuhip_fc_prepack packs matrices of few rows
  if (w->algo != ALGO_MFMA || !d.relu_first || d.ih != 1 || d.iw != 1 || w->split_oc ||
      std::string(kTiles[w->tile].name) != "mfma_reg_32x32")
    return false;
  const int n_pb = (d.n + 31) / 32, n_ob = w->ocp / 32, nsteps = w->kp / 64;
  p->tiles = n_pb * n_ob;
  if (p->tiles > kFcMaxTiles) return false;
  // about two waves per CU of the chip, at least two K steps each
  const int want = std::max(1, ctx->num_cu * 2 / p->tiles);
  p->splits = std::max(1, std::min(want, nsteps / 2));
  p->steps_per_split = (nsteps + p->splits - 1) / p->splits;
  p->splits = (nsteps + p->steps_per_split - 1) / p->steps_per_split;
  p->bytes = (size_t)p->tiles * p->splits * kFcPartialBytes;
  return true;
}

static int run_fc_splitk(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y, void *scratch_ptr,
                         const FcPlan &p) {
  ConvArgs a;
  fill_args(ctx, w, x, y, &a);
  a.n_oc_tiles = w->ocp / 32;
  // with per-kernel profiling events set, the pair brackets both launches: begin of the first,
  // end of the second
  const dim3 grid1((unsigned)(p.tiles * p.splits)), grid2((unsigned)p.tiles);
  v4i *parts = (v4i *)scratch_ptr;
  if (ctx->prof_start)
    hipExtLaunchKernelGGL(fc_partial_kernel, grid1, dim3(64), 0, ctx->stream, ctx->prof_start, nullptr, 0, a, parts,
                          p.splits, p.steps_per_split);
  else
    hipLaunchKernelGGL(fc_partial_kernel, grid1, dim3(64), 0, ctx->stream, a, parts, p.splits, p.steps_per_split);
  auto reduce = w->fast ? fc_reduce_kernel<true> : fc_reduce_kernel<false>;
  if (ctx->prof_stop)
    hipExtLaunchKernelGGL(reduce, grid2, dim3(256), 0, ctx->stream, nullptr, ctx->prof_stop, 0, a, (const v4i *)parts,
                          p.splits);
  else
    hipLaunchKernelGGL(reduce, grid2, dim3(256), 0, ctx->stream, a, (const v4i *)parts, p.splits);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

static int run_fc_one(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y) {
  ConvArgs a;
  fill_args(ctx, w, x, y, &a);
  a.n_oc_tiles = w->ocp / 32;
  const int nsteps = w->kp / 64;
  const int64_t tiles = (int64_t)((w->d.n + 31) / 32) * a.n_oc_tiles;
  TPUHIP_REQUIRE(tiles < (1ll << 31), "fc: too many blocks of 32 x 32 outputs");
  const int steps_per_wave = (nsteps + kFcOneWaves - 1) / kFcOneWaves;
  auto kernel = w->fast ? fc_one_kernel<true> : fc_one_kernel<false>;
  const dim3 grid((unsigned)tiles), block(64 * kFcOneWaves);
  if (ctx->prof_start || ctx->prof_stop)
    hipExtLaunchKernelGGL(kernel, grid, block, 0, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a, steps_per_wave);
  else
    hipLaunchKernelGGL(kernel, grid, block, 0, ctx->stream, a, steps_per_wave);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

// a context that goes away is forgotten as the static scratch's last user (its stream handle dies with it)
void tpuhip_static_scratch_forget(const tpuhip_ctx *ctx) {
  std::lock_guard<std::mutex> lock(g_static_mu);
  for (int d = 0; d < 64; ++d)
    if (g_static_user[d] == ctx) {
      g_static_user[d] = nullptr;
      g_static_stream[d] = nullptr;
    }
}

int tpuhip_static_scratch_init(int device) {
  TPUHIP_REQUIRE(device >= 0 && device < 64, "tpuhip: device index %d out of range", device);
  if (g_static_scratch[device]) return TPUHIP_OK;
  void *ptr = nullptr;
  TPUHIP_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  g_static_scratch[device] = ptr;
  return TPUHIP_OK;
}

int tpuhip_fc_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && w && x && y, "tpuhip_fc_i8: NULL argument");
  FcPlan p;
  if (!fc_splitk_plan(ctx, w, &p)) return run_conv(ctx, w, x, y, PostOps{});   // many rows: the conv path
  if (w->kp / 64 >= kFcOneWaves) return run_fc_one(ctx, w, x, y);              // long K: one launch
  if (ctx->workspace_bytes < p.bytes) {
    TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
    TPUHIP_CHECK_HIP(hipStreamSynchronize(ctx->stream));
    if (ctx->workspace) TPUHIP_CHECK_HIP(hipFree(ctx->workspace));
    ctx->workspace = nullptr;
    ctx->workspace_bytes = 0;
    TPUHIP_CHECK_HIP(hipMalloc(&ctx->workspace, p.bytes));
    ctx->workspace_bytes = p.bytes;
  }
  return run_fc_splitk(ctx, w, x, y, ctx->workspace, p);
}

int tpuhip_fc_i8_noalloc(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && w && x && y, "tpuhip_fc_i8_noalloc: NULL argument");
  FcPlan p;
  TPUHIP_REQUIRE(fc_splitk_plan(ctx, w, &p),
                 "tpuhip_fc_i8_noalloc: not a FullyConnected packed by tpuhip_fc_prepack for the split-K kernel "
                 "(at most 256 rows, at most %d blocks of 32 x 32 outputs)", kFcMaxTiles);
  TPUHIP_REQUIRE(p.bytes <= kFcStaticBytes,
                 "tpuhip_fc_i8_noalloc: the layer needs %zu bytes of scratch, the static buffer holds %zu "
                 "(%zu partial sums of 32 x 32 outputs)", p.bytes, kFcStaticBytes, kFcStaticPartials);
  void *ptr = ctx->device >= 0 && ctx->device < 64 ? g_static_scratch[ctx->device] : nullptr;
  TPUHIP_REQUIRE(ptr, "tpuhip_fc_i8_noalloc: the static scratch of device %d was not set up", ctx->device);
  {
    std::lock_guard<std::mutex> lock(g_static_mu);
    const tpuhip_ctx *last = g_static_user[ctx->device];
    if (last && last != ctx && g_static_stream[ctx->device] != ctx->stream) {
      // (a query, no wait: the call stays free of anything that blocks or allocates)
      const hipError_t q = hipStreamQuery(g_static_stream[ctx->device]);
      if (q == hipErrorNotReady)
        return set_error(TPUHIP_ERR_INVALID,
                         "tpuhip_fc_i8_noalloc: another context's call on device %d is still in flight on its "
                         "stream; calls that overlap on one GPU share the static scratch and would race",
                         ctx->device);
      (void)hipGetLastError();
    }
    g_static_user[ctx->device] = ctx;
    g_static_stream[ctx->device] = ctx->stream;
  }
  return run_fc_splitk(ctx, w, x, y, ptr, p);
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
  // few rows: packed fragment by fragment for the split-K kernel of tpuhip_fc_i8 (the same
  // bytes serve the LDS-free 32x32 conv tile, so tpuhip_conv2d_i8 runs them too)
  // (and so is a K beyond the conv kernels' reach, whatever the rows)
  if ((m <= 256 && (n + 31) / 32 * ((m + 31) / 32) <= kFcMaxTiles) || k > 4096) {
    for (int t = 0; t < kNumTiles; ++t)
      if (std::string(kTiles[t].name) == "mfma_reg_32x32") d.algo = 16 + t;
  }
  std::vector<int32_t> mult((size_t)n, multiplier), rs((size_t)n, rshift);
  return tpuhip_conv2d_prepack(ctx, &d, filter_nk, bias, mult.data(), rs.data(), out);
}

}  // extern "C"

// A depthwise convolution (at most 3 x 3 taps) and the pointwise convolution that reads its result,
// as one launch -- the second half of an inverted-residual block (MobileNet): depthwise + ReLU,
// optionally a 256-entry table (ReLU6 / clip), 1x1 projection, optionally the block's residual add.
//
//   Conv2DOpKernel::invoke (core/conv.cpp:11-104, the g != 1 branch) for the depthwise conv,
//   LutOpKernel (core/activation.cpp:47-53, core/clip.cpp:29-40) on its result, Conv2DOpKernel::invoke
//   for the 1x1 conv, EltwiseAddOpKernel::i8_invoke (core/eltwise.cpp:52-85) on (add_src, its result)
//   -- the same bytes as the ops run one after the other.
//
// The depthwise result -- the widest tensor of the block -- is not read back from memory (and not
// written either, unless the caller keeps it).  Both convs run on the matrix cores:
//   * phase 1, depthwise: a tap is a 32x32 DIAGONAL matrix times the 32 channels x 32 pixels
//     activation block, one v_mfma_i32_32x32x32_i8 per tap.  A wave's 32 pixels are R row segments
//     of W lanes of one image; with 3 taps along W at stride 1 a lane loads only the middle tap of
//     each filter row and takes the outer two from its neighbours (DPP), the first and last lane of
//     a segment being halo.  A lane's 16 results are 16 consecutive channels of its pixel: after
//     the requantisation they are four dwords, which is exactly the B-operand fragment of the 1x1
//     conv's MFMA for that 32-channel K slice.  They go to LDS in that form.
//   * phase 2, pointwise: the workgroup's P pixel blocks x (output channels / 32) result blocks
//     are dealt to the four waves -- or, where there are fewer than four, a result block's K slices
//     are split between waves and the parts added up in LDS (integer adds: any order, same sum).  A
//     wave requests the A fragments (the 1x1 filter, packed in fragment order) of up to eight K
//     slices at a time from global memory, takes the B fragments from LDS, then requantises, adds the
//     residual and stores 16 bytes per lane.
// A workgroup owns P consecutive pixel blocks (P = 4 for narrow 1x1 convs, down to 1 for wide ones);
// the waves split the (K slice, pixel block) items of phase 1 in K-slice-major order, so a wave reloads
// its nine diagonal fragments once per P items.  The first item's input is requested before the data the
// workgroup shares (the 1x1 conv's requantisation planes, the table) is copied to LDS.
//
// Measured on MobileNetV2's blocks at batch 64 the launch is within +-10 % of the two launches it
// replaces on maps of 14 x 14 to 56 x 56 and slower on 7 x 7 maps and on 1x1 convs of more than 96
// channels: both forms issue about nine vector instructions per depthwise output (requantisation,
// neighbour-lane moves, addresses) and that, not the memory traffic saved, bounds them.  Callers
// choose per layer pair; the graph interpreter does not chain depthwise convs by itself.
#include "conv_chain.hpp"

#include <algorithm>
#include <cstring>

using namespace tpuhip;

struct DwPwArgs {
  const int8_t *x;         // [n][ih][iw][x_cs]
  const int8_t *wdw;       // diagonal A fragments [32-channel block][9][lane][16]
  const int32_t *qdw;      // per 32-channel block 160 words: 32 (low, high) addends | 32 mult | 32 shift | 32 2^(r-1)
  const int8_t *wpw;       // A fragments of the 1x1 filter [32-channel block][K slice][lane][16]
  const int32_t *qpw;      // planes of 32 * n_tm channels: addends | mult | shift | 2^(r-1)
  int8_t *y_dw;            // the depthwise result, or null
  int8_t *lut_dst;         // table[depthwise result], or null
  const int8_t *add_src;   // the residual, or null
  int8_t *add_dst;         // the sum, or null
  int8_t *y;               // the 1x1 result, or null (then the sum is what the caller wants)
  uint32_t x_bytes;
  int ih, iw, x_cs, oh, ow;
  int c, cw, mid_cs;       // depthwise channels, rounded up to 16, channel stride of y_dw / lut_dst
  int ocw, y_cs;           // 1x1 output channels rounded up to 16, channel stride of y / add_src / add_dst
  int kh, kw, sh, sw, pt, pl, dh, dw;
  int relu_dw, relu_pw;
  int add_m_src, add_m_conv, add_rshift, add_relu, add_pk;
  int has_lut;
  Table256 lut;
  int rows, width, valid, halo;      // R, W, outputs per row segment (W - 2 * halo)
  int xblocks, rblocks, nblocks;     // column blocks per output row, row blocks per image, n * rblocks * xblocks
  uint32_t magic_w;                  // ceil(2^32 / width)
  int log2p, n_cb, n_tm, ngroups;    // P = 1 << log2p pixel blocks per workgroup
  int nk;                            // phase 2: waves that split the K slices of one result block
};

template <bool SHIFT, int NT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(SHIFT ? 4 : 3, SHIFT ? 4 : 3))) void
conv_dwpw_kernel(DwPwArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int P = 1 << a.log2p;
  const int ocp = a.n_tm * 32;
  v4i *bfr = reinterpret_cast<v4i *>(smem);                                    // [P][n_cb][64 lanes]
  int32_t *q2 = reinterpret_cast<int32_t *>(smem + (size_t)P * a.n_cb * 1024);   // the 1x1 conv's planes
  int32_t *qall = q2 + 5 * ocp;                                                // [4 waves][160]
  uint32_t *lutw = reinterpret_cast<uint32_t *>(qall + 4 * 160);
  int32_t *red = reinterpret_cast<int32_t *>(lutw + 64);                        // [result block][16][64] when nk > 1
  const int tiles = a.n_tm << a.log2p;

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int p32 = lane & 31, fk = lane >> 5;
  // workgroups are dealt to the 8 XCDs round-robin; each XCD takes a contiguous run of groups, so the
  // input rows that vertically neighbouring blocks share meet in one L2
  const int per_xcd = (a.ngroups + 7) >> 3;
  const int xcd = (int)(blockIdx.x & 7);
  const int g = xcd * per_xcd + (int)(blockIdx.x >> 3);
  if (g >= a.ngroups || g >= (xcd + 1) * per_xcd) return;   // the whole workgroup: no barrier is missed
  const int b0 = g << a.log2p;
  const int nb = min(P, a.nblocks - b0);                    // pixel blocks of this group that exist

  const uint8_t *lut = a.has_lut ? reinterpret_cast<const uint8_t *>(lutw) : nullptr;

  // block b0 -> (image, row block, column block); the next ones follow with carries
  int xb0, rb0, n0;
  {
    const int t = b0 / a.xblocks;
    xb0 = b0 - t * a.xblocks;
    n0 = t / a.rblocks;
    rb0 = t - n0 * a.rblocks;
  }
  auto block_coords = [&](int p, int &n, int &rb, int &xb) {
    xb = xb0 + p;
    rb = rb0;
    n = n0;
    while (xb >= a.xblocks) { xb -= a.xblocks; ++rb; }      // at most P - 1 trips
    while (rb >= a.rblocks) { rb -= a.rblocks; ++n; }
  };

  // what never changes for a lane
  const int lr = (int)__umulhi((uint32_t)p32, a.magic_w), lc = p32 - lr * a.width;
  const bool in_block = p32 < a.rows * a.width;
  const bool inner = in_block & (lc >= a.halo) & (lc < a.halo + a.valid);
  const int lrow_in = lr * a.sh;
  const int lcol_in = (lc - a.halo) * a.sw - a.pl + (SHIFT ? 1 : 0);
  const int row_bytes = a.iw * a.x_cs, drow_bytes = a.dh * row_bytes;
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);

  // ---- phase 1: depthwise ------------------------------------------------
  {
    int32_t *qw = qall + wave * 160;
    const int32_t *pc64 = qw + fk * 32, *pmult = qw + 64 + fk * 16, *pshift = qw + 96 + fk * 16, *phpot = qw + 128 + fk * 16;
    const int T = a.n_cb << a.log2p;
    const int chunk = (T + 3) >> 2;
    int it = wave * chunk;
    const int it_end = min(T, it + chunk);
    int cur_cb = -1;
    v4i areg[3][3], bt[3][3];

    auto request = [&](int cb, int p) {
      int n, rb, xb;
      block_coords(p, n, rb, xb);
      const int oc = cb * 32 + fk * 16;
      const bool live = in_block & (oc < a.cw) & (p < nb);
      const int ihb = rb * a.rows * a.sh - a.pt + lrow_in;
      const int iw0 = xb * a.valid * a.sw + lcol_in;
      const uint32_t img_base = (uint32_t)n * (uint32_t)(a.ih * row_bytes);
      // rows and row pitch are below 2^23 (checked on the host); a first row above the image gives a
      // negative product, from which the rows below it are still reached
      const uint32_t off0 = (uint32_t)__mul24(ihb, row_bytes) + (uint32_t)(iw0 * a.x_cs + oc);
      if (SHIFT) {
        const bool col_ok = live & ((unsigned)iw0 < (unsigned)a.iw);
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

    if (it < it_end) request(it >> a.log2p, it & (P - 1));
    // what the whole workgroup shares goes to LDS while the first input is on its way
    for (int i = threadIdx.x; i < 5 * ocp; i += 256) q2[i] = a.qpw[i];
    if (a.has_lut && threadIdx.x < 64) lutw[threadIdx.x] = a.lut.w[threadIdx.x];
    if (a.nk > 1)
      for (int i = threadIdx.x; i < tiles * 1024; i += 256) red[i] = 0;
    __syncthreads();
    while (it < it_end) {
      const int cb = it >> a.log2p, p = it & (P - 1);
      if (cb != cur_cb) {
        // this wave's nine diagonal fragments and requantisation data of the K slice
        const v4i *afrag = reinterpret_cast<const v4i *>(a.wdw) + (size_t)cb * 9 * 64 + lane;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
          for (int j = 0; j < 3; ++j)
            areg[i][j] = (i < a.kh && j < a.kw) ? afrag[(i * a.kw + j) * 64] : v4i{0, 0, 0, 0};
        const int32_t *src = a.qdw + (size_t)cb * 160;
        qw[lane] = src[lane];
        qw[64 + lane] = src[64 + lane];
        if (lane < 32) qw[128 + lane] = src[128 + lane];
        cur_cb = cb;
      }
      v16i acc[1];
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[0][e] = 0;
#pragma unroll
      for (int i = 0; i < 3; ++i) {
        if (SHIFT) {
          bt[i][0] = shift_lanes(bt[i][1], 0);
          bt[i][2] = shift_lanes(bt[i][1], 1);
        }
#pragma unroll
        for (int j = 0; j < 3; ++j)
          acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(areg[i][j], bt[i][j], acc[0], 0, 0, 0);
      }
      // where this item's results go, before the walk moves on
      int n, rb, xb;
      block_coords(p, n, rb, xb);
      const int oh = rb * a.rows + lr, ow = xb * a.valid + lc - a.halo;
      const int oc = cb * 32 + fk * 16;
      const bool st_ok = inner & (p < nb) & (oh < a.oh) & (ow < a.ow) & (oc < a.cw);
      const int64_t off = ((int64_t)(n * a.oh + oh) * a.ow + ow) * a.mid_cs + oc;
      ++it;
      // the next item's input goes into the registers the MFMAs have just consumed -- unless it
      // belongs to another K slice: its fragments are fetched first, at the top of the loop
      if (it < it_end) request(it >> a.log2p, it & (P - 1));
      uint32_t outw[1][4];
      if (a.relu_dw) requant_rows_c64<1, true>(acc, 0, pc64, pmult, pshift, phpot, outw);
      else requant_rows_c64<1, false>(acc, -128, pc64, pmult, pshift, phpot, outw);
      v4i o = {(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
      if (a.y_dw && st_ok) *reinterpret_cast<v4i *>(a.y_dw + off) = o;
      if (lut) {
        // table lookup per byte; pad channels stay zero whatever table[0] is
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t wd = (uint32_t)o[q];
          const uint32_t r = (uint32_t)lut[wd & 255u] | ((uint32_t)lut[(wd >> 8) & 255u] << 8) |
                             ((uint32_t)lut[(wd >> 16) & 255u] << 16) | ((uint32_t)lut[wd >> 24] << 24);
          const int valid = a.c - (oc + q * 4);
          const uint32_t mask = valid >= 4 ? 0xffffffffu : valid <= 0 ? 0u : (1u << (8 * valid)) - 1u;
          o[q] = (int)(r & mask);
        }
        if (a.lut_dst && st_ok) *reinterpret_cast<v4i *>(a.lut_dst + off) = o;
      }
      bfr[(p * a.n_cb + cb) * 64 + lane] = o;
    }
  }
  __syncthreads();

  // ---- phase 2: pointwise --------------------------------------------------
  {
    // a unit of work: (result block t, part kp of its K slices); result block t -> (channel block t >> log2p,
    // pixel block t & (P - 1)).  nk > 1: wave w takes block w % tiles, part w / tiles, and the parts meet in
    // LDS; nk == 1: wave w takes blocks w, w + 4, ...
    int tl[NT], tm[NT], pp[NT];
    bool on[NT];
    const int kp = a.nk > 1 ? wave / tiles : 0;
    const int kper = (a.n_cb + a.nk - 1) / a.nk;
    const int k0 = kp * kper, k1 = min(a.n_cb, k0 + kper);
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      tl[i] = a.nk > 1 ? wave - kp * tiles : wave + 4 * i;
      tm[i] = tl[i] >> a.log2p;
      pp[i] = tl[i] & (P - 1);
      on[i] = (tl[i] < tiles) & (pp[i] < nb) & (kp < a.nk) & (a.nk == 1 || i == 0);
    }
    v16i acc2[NT][1];
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc2[i][0][e] = 0;
    const v4i *wfrag = reinterpret_cast<const v4i *>(a.wpw) + lane;
    constexpr int U = NT == 1 ? 8 : NT == 2 ? 4 : 2;      // K slices whose A fragments are requested together
    for (int kb = k0; kb < k1; kb += U) {
      v4i af[NT][U];
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int u = 0; u < U; ++u) {
          af[i][u] = v4i{0, 0, 0, 0};
          if (on[i] && kb + u < k1) af[i][u] = wfrag[(size_t)(tm[i] * a.n_cb + kb + u) * 64];
        }
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int i = 0; i < NT; ++i)
          if (on[i] && kb + u < k1)
            acc2[i][0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af[i][u], bfr[(pp[i] * a.n_cb + kb + u) * 64 + lane],
                                                                acc2[i][0], 0, 0, 0);
    }
    if (a.nk > 1) {
      // the parts of a result block are summed in LDS (integer adds: any order gives the same sum)
      if (on[0]) {
#pragma unroll
        for (int e = 0; e < 16; ++e) atomicAdd(&red[(tl[0] * 16 + e) * 64 + lane], acc2[0][0][e]);
      }
      __syncthreads();
      if (on[0] && kp == 0) {
#pragma unroll
        for (int e = 0; e < 16; ++e) acc2[0][0][e] = red[(tl[0] * 16 + e) * 64 + lane];
      }
#pragma unroll
      for (int i = 0; i < NT; ++i) on[i] = on[i] & (kp == 0);
    }
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      if (!on[i]) continue;
      int n, rb, xb;
      block_coords(pp[i], n, rb, xb);
      const int oh = rb * a.rows + lr, ow = xb * a.valid + lc - a.halo;
      const int oc = tm[i] * 32 + fk * 16;
      const bool st_ok = inner & (oh < a.oh) & (ow < a.ow) & (oc < a.ocw);
      const int64_t off = ((int64_t)(n * a.oh + oh) * a.ow + ow) * a.y_cs + oc;
      v4i sv = {0, 0, 0, 0};
      if (a.add_dst && st_ok) sv = *reinterpret_cast<const v4i *>(a.add_src + off);
      uint32_t outw[1][4];
      if (a.relu_pw) requant_rows_c64<1, true>(acc2[i], 0, q2 + 2 * oc, q2 + 2 * ocp + oc, q2 + 3 * ocp + oc, q2 + 4 * ocp + oc, outw);
      else requant_rows_c64<1, false>(acc2[i], -128, q2 + 2 * oc, q2 + 2 * ocp + oc, q2 + 3 * ocp + oc, q2 + 4 * ocp + oc, outw);
      if (st_ok) {
        const v4i o = {(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
        if (a.y) *reinterpret_cast<v4i *>(a.y + off) = o;
        if (a.add_dst)
          *reinterpret_cast<v4i *>(a.add_dst + off) =
              fused_add_chunk(o, sv, a.add_m_src, a.add_m_conv, a.add_rshift, a.add_relu, a.add_pk);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
namespace {

struct DwPwPlan {
  int rows, width, valid, halo, xblocks, rblocks, nblocks;
  int n_cb, n_tm, log2p, nt, nk;
};

// the row segments of the depthwise phase (fewest blocks per image) and the pixel blocks per workgroup
bool dwpw_plan(const tpuhip_conv_desc &a, const tpuhip_conv_desc &b, DwPwPlan *out) {
  const bool depthwise = a.g == a.ic && a.g == a.oc && a.g > 1 && !a.ins_h && !a.ins_w && !a.relu_first;
  if (!depthwise || a.kh < 1 || a.kw < 1 || a.kh > 3 || a.kw > 3) return false;
  if (!is_pointwise_conv(b) || b.n != a.n || b.ih != a.oh || b.iw != a.ow || b.ic != a.oc || b.x_cs != a.y_cs) return false;
  if (a.x_cs % 16 || a.y_cs % 16 || b.y_cs % 16 || a.x_cs < a.ic || a.y_cs < a.oc || b.y_cs < b.oc) return false;
  if (a.sh < 1 || a.sw < 1 || a.dh < 1 || a.dw < 1 || a.sh > 4 || a.sw > 4 || a.pl > 64 || a.pt > 64) return false;
  // input rows and the row pitch fit the 24-bit multiply of the address arithmetic; 32-bit byte offsets
  if (a.ih >= (1 << 22) || (int64_t)a.iw * a.x_cs >= (1ll << 23)) return false;
  if ((int64_t)a.n * a.ih * a.iw * a.x_cs >= (1ll << 31) || (int64_t)a.n * a.oh * a.ow * a.y_cs >= (1ll << 31) ||
      (int64_t)b.n * b.oh * b.ow * b.y_cs >= (1ll << 31))
    return false;
  const int halo = (a.kw == 3 && a.sw == 1 && a.dw == 1) ? 1 : 0;
  int64_t best = -1;
  for (int rows = 1; rows <= 4; ++rows) {
    const int width = 32 / rows, valid = width - 2 * halo;
    if (valid < 1) continue;
    const int64_t blocks = (int64_t)((a.oh + rows - 1) / rows) * ((a.ow + valid - 1) / valid);
    if (best < 0 || blocks < best) {
      best = blocks;
      out->rows = rows; out->width = width; out->valid = valid; out->halo = halo;
      out->rblocks = (a.oh + rows - 1) / rows;
      out->xblocks = (a.ow + valid - 1) / valid;
    }
  }
  if (best < 0 || best * a.n >= (1ll << 28)) return false;
  out->nblocks = (int)(best * a.n);
  out->n_cb = (a.oc + 31) / 32;
  out->n_tm = (b.oc + 31) / 32;
  if (out->n_cb > 60 || out->n_tm > 12) return false;
  // pixel blocks per workgroup: a result block for every wave of phase 2 where the 1x1 conv is narrow,
  // within 60 KB of B fragments, and no fewer than about two workgroups per CU's worth of groups
  int log2p = out->n_tm == 1 ? 2 : out->n_tm <= 3 ? 1 : 0;
  while (log2p > 0 && ((out->n_cb << log2p) > 60 || (out->nblocks >> log2p) < 512)) --log2p;
  out->log2p = log2p;
  out->nt = ((out->n_tm << log2p) + 3) / 4;
  const int tiles = out->n_tm << log2p;
  out->nk = tiles < 4 ? std::min(4 / tiles, out->n_cb) : 1;
  return out->nt <= 3;
}

std::vector<int8_t> diagonal_fragments(const int8_t *filter, int c, int n_cb, int kh, int kw) {
  // [32-channel block][9][lane][16 bytes]; lane l holds row l & 31 (channel mfma_row_to_oc(row) of
  // the block), K bytes 16 * (l >> 5) .. + 15: one weight on the diagonal, zeros elsewhere
  const int taps = kh * kw;
  std::vector<int8_t> out((size_t)n_cb * 9 * 1024, 0);
  for (int cb = 0; cb < n_cb; ++cb)
    for (int t = 0; t < taps; ++t)
      for (int lane = 0; lane < 64; ++lane) {
        const int ch_in_block = mfma_row_to_oc(lane & 31, 1);
        const int ch = cb * 32 + ch_in_block;
        const int j = ch_in_block - 16 * (lane >> 5);
        if (ch < c && j >= 0 && j < 16) out[((size_t)(cb * 9 + t) * 64 + lane) * 16 + j] = filter[(size_t)ch * taps + t];
      }
  return out;
}

const char *const kDwPwNames[] = {"mfma_dwpw_shift_nt1", "mfma_dwpw_shift_nt2", "mfma_dwpw_shift_nt3",
                                  "mfma_dwpw_taps_nt1",  "mfma_dwpw_taps_nt2",  "mfma_dwpw_taps_nt3"};

unsigned dwpw_lds_bytes(const DwPwPlan &p) {
  return (unsigned)(((size_t)p.n_cb << p.log2p) * 1024 + (size_t)5 * p.n_tm * 32 * 4 + 4 * 160 * 4 + 256 +
                    (p.nk > 1 ? ((size_t)p.n_tm << p.log2p) * 4096 : 0));
}

}  // namespace

namespace tpuhip {

const char *dwpw_variant_name(int i) { return i >= 0 && i < 6 ? kDwPwNames[i] : nullptr; }

bool dwpw_covers(const tpuhip_conv_desc &a, const tpuhip_conv_desc &b) {
  DwPwPlan p;
  return dwpw_plan(a, b, &p);
}

int dwpw_prepack(tpuhip_ctx *ctx, tpuhip_conv_chain *ch, const int8_t *filter_a, const int32_t *bias_a,
                 const int32_t *mult_a, const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                 const int32_t *mult_b, const int32_t *rshift_b) {
  const tpuhip_conv_desc &a = ch->da, &b = ch->db;
  DwPwPlan p;
  if (!dwpw_plan(a, b, &p)) return set_error(TPUHIP_ERR_UNSUPPORTED, "conv chain: shapes not covered");
  std::vector<int32_t> pa, pb;
  const int cp = p.n_cb * 32, ocp = p.n_tm * 32;
  if (!requant_planes(a.oc, cp, (size_t)a.kh * a.kw, a.do_relu != 0, filter_a, (a.with_bias && bias_a) ? bias_a : nullptr,
                      mult_a, rshift_a, &pa) ||
      !requant_planes(b.oc, ocp, (size_t)b.ic, b.do_relu != 0, filter_b, (b.with_bias && bias_b) ? bias_b : nullptr, mult_b,
                      rshift_b, &pb))
    return set_error(TPUHIP_ERR_UNSUPPORTED,
                     "conv chain: needs right shifts of at least 1 and sums that cannot overflow the rounding");
  // the depthwise planes, regrouped per 32-channel block: 32 addend pairs | 32 mult | 32 shift | 32 2^(r-1)
  std::vector<int32_t> qa((size_t)p.n_cb * 160, 0);
  for (int cb = 0; cb < p.n_cb; ++cb)
    for (int i = 0; i < 32; ++i) {
      const int chn = cb * 32 + i;
      int32_t *q = qa.data() + (size_t)cb * 160;
      q[2 * i] = pa[2 * chn];
      q[2 * i + 1] = pa[2 * chn + 1];
      q[64 + i] = pa[2 * cp + chn];
      q[96 + i] = pa[3 * cp + chn];
      q[128 + i] = pa[4 * cp + chn];
    }
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const std::vector<int8_t> f1 = diagonal_fragments(filter_a, a.oc, p.n_cb, a.kh, a.kw);
  const std::vector<int8_t> f2 = mfma_a_fragments(filter_b, b.oc, p.n_tm, b.ic, cp, 1);
  int rc = upload_vec(ctx, f1, &ch->w1);
  if (!rc) rc = upload_vec(ctx, f2, &ch->w2);
  if (!rc) rc = upload_vec(ctx, qa, &ch->q1);
  if (!rc) rc = upload_vec(ctx, pb, &ch->q2);
  ch->variant = (p.halo ? 0 : 3) + p.nt - 1;
  ch->name = kDwPwNames[ch->variant];
  return rc;
}

int dwpw_run(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y_a, const tpuhip_conv_post *post_a,
             void *y_b, const tpuhip_conv_post *post_b) {
  const tpuhip_conv_desc &da = ch->da, &db = ch->db;
  DwPwPlan p;
  TPUHIP_REQUIRE(dwpw_plan(da, db, &p), "conv chain: shapes not covered");
  TPUHIP_REQUIRE(!(post_a && post_a->add.enable), "conv chain: a depthwise -> pointwise chain takes no add behind the first conv");
  TPUHIP_REQUIRE(!(post_b && post_b->lut), "conv chain: a depthwise -> pointwise chain takes no table behind the second conv");
  const bool add = post_b && post_b->add.enable;
  TPUHIP_REQUIRE(!add || (post_b->add_src && post_b->add_out), "conv chain: fused add without its operand or result");
  TPUHIP_REQUIRE(y_b || add, "conv chain: nothing to write");
  DwPwArgs a{};
  a.x = (const int8_t *)x;
  a.wdw = ch->w1;
  a.qdw = ch->q1;
  a.wpw = ch->w2;
  a.qpw = ch->q2;
  a.y_dw = (int8_t *)y_a;
  a.y = (int8_t *)y_b;
  if (post_a && post_a->lut) {
    a.has_lut = 1;
    std::memcpy(a.lut.w, post_a->lut, 256);
    a.lut_dst = (int8_t *)post_a->lut_out;
  }
  if (add) {
    const tpuhip_fused_add &f = post_b->add;
    TPUHIP_REQUIRE(f.rshift >= 0 && f.rshift <= 30, "conv chain: add rshift %d outside [0,30]", f.rshift);
    TPUHIP_REQUIRE(f.m_src >= -128 && f.m_src <= 127 && f.m_conv >= -128 && f.m_conv <= 127,
                   "conv chain: add multipliers must be int8");
    a.add_src = (const int8_t *)post_b->add_src;
    a.add_dst = (int8_t *)post_b->add_out;
    a.add_m_src = f.m_src;
    a.add_m_conv = f.m_conv;
    a.add_rshift = f.rshift;
    a.add_relu = f.do_relu ? 1 : 0;
    a.add_pk = std::abs(f.m_src) <= 127 && std::abs(f.m_conv) <= 127 && f.rshift <= 8;
  }
  a.x_bytes = (uint32_t)((int64_t)da.n * da.ih * da.iw * da.x_cs);
  a.ih = da.ih; a.iw = da.iw; a.x_cs = da.x_cs; a.oh = da.oh; a.ow = da.ow;
  a.c = da.oc; a.cw = (da.oc + 15) / 16 * 16; a.mid_cs = da.y_cs;
  a.ocw = (db.oc + 15) / 16 * 16; a.y_cs = db.y_cs;
  a.kh = da.kh; a.kw = da.kw; a.sh = da.sh; a.sw = da.sw; a.pt = da.pt; a.pl = da.pl; a.dh = da.dh; a.dw = da.dw;
  a.relu_dw = da.do_relu ? 1 : 0;
  a.relu_pw = db.do_relu ? 1 : 0;
  a.rows = p.rows; a.width = p.width; a.valid = p.valid; a.halo = p.halo;
  a.xblocks = p.xblocks; a.rblocks = p.rblocks; a.nblocks = p.nblocks;
  a.magic_w = p.width > 1 ? (uint32_t)(((1ull << 32) + p.width - 1) / (uint64_t)p.width) : 0u;
  a.log2p = p.log2p; a.n_cb = p.n_cb; a.n_tm = p.n_tm; a.nk = p.nk;
  a.ngroups = (p.nblocks + (1 << p.log2p) - 1) >> p.log2p;
  const unsigned lds = dwpw_lds_bytes(p);
  const dim3 grid(8u * (unsigned)((a.ngroups + 7) / 8)), block(256);
#define TPUHIP_DWPW_LAUNCH(SH, NTV)                                                                       \
  {                                                                                                       \
    auto kernel = conv_dwpw_kernel<SH, NTV>;                                                              \
    TPUHIP_REQUIRE(raise_dynamic_lds((const void *)kernel, lds), "conv chain: raising the LDS limit failed"); \
    if (ctx->prof_start)                                                                                  \
      hipExtLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                  \
      hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, a);                                       \
  }
  if (p.halo) {
    if (p.nt == 1) TPUHIP_DWPW_LAUNCH(true, 1) else if (p.nt == 2) TPUHIP_DWPW_LAUNCH(true, 2) else TPUHIP_DWPW_LAUNCH(true, 3)
  } else {
    if (p.nt == 1) TPUHIP_DWPW_LAUNCH(false, 1) else if (p.nt == 2) TPUHIP_DWPW_LAUNCH(false, 2) else TPUHIP_DWPW_LAUNCH(false, 3)
  }
#undef TPUHIP_DWPW_LAUNCH
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // namespace tpuhip

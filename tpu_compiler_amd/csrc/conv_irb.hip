// An inverted-residual block as one launch: the 1x1 expansion, the depthwise conv (at most 3 x 3 taps)
// behind it and the 1x1 projection behind that, with the block's residual add (MobileNetV2).
//
//   Conv2DOpKernel::invoke three times (core/conv.cpp:11-104; the g != 1 branch for the middle one)
//   and EltwiseAddOpKernel::i8_invoke (core/eltwise.cpp:52-85) on (add_src, the projection's result)
//   -- the same bytes as the ops run one after the other.
//
// The two expanded tensors -- six times as wide as the block's input and output -- never leave the
// chip.  A workgroup owns P vertically neighbouring pixel blocks (R rows x W pixels each, R * W <= 32)
// of one image and runs three phases, all on the matrix cores:
//   * expansion: the input pixels under the blocks' windows (a patch of prows x pcols pixels, halo
//     included; fetched into LDS once by the whole workgroup, pixels outside the image as zeros) times
//     the expansion filter: patch pixels are MFMA columns, 32-channel blocks of the filter are A
//     fragments, dealt to the waves.  Requantised results go to an LDS patch
//     [pixel][channels], pixel pitch an odd number of 16-byte chunks; pixels outside the image are
//     stored as ZEROS -- the depthwise conv pads its input, the expansion's result, with zeros.
//   * depthwise: a tap is a 32x32 diagonal matrix times 32 channels x 32 pixels read from the patch
//     at the tap's offset; the diagonal fragments are built from one dword per lane and tap.  A
//     lane's 16 requantised channels are the B fragment of the projection's MFMA for that K slice and
//     go to LDS as such.
//   * projection: result blocks (32 channels x 32 pixels) dealt to the waves, or their K slices split
//     between idle waves and summed in LDS; A fragments from global memory eight slices at a time;
//     requantisation, residual add, 16-byte stores.
// The halo pixels of the expansion are computed by every workgroup that needs them (a 2 x 16 block of
// a 14 x 14 map expands 4 x 18 pixels): the expansion is the cheapest of the three convs, and what it
// buys is two launches and four passes over the widest tensors of the network.
#include "conv_chain.hpp"

#include <algorithm>
#include <cstring>

using namespace tpuhip;

constexpr int kIrbMaxKsIn = 5;   // the expansion's input: at most 160 channels

struct IrbArgs {
  const int8_t *x;         // [n][ih][iw][x_cs]
  const int8_t *wex;       // expansion: A fragments [32-channel block][K slice][lane][16]
  const int32_t *qex;      // per 32-channel block 160 words: 32 (low, high) addends | 32 mult | 32 shift | 32 2^(r-1)
  const uint32_t *wdw;     // depthwise: [32-channel block][9][lane] the lane's dword of the diagonal fragment
  const int32_t *qdw;      // as qex
  const int8_t *wpw;       // projection: A fragments [32-channel block][K slice][lane][16]
  const int32_t *qpw;      // planes of 32 * n_tm channels: addends | mult | shift | 2^(r-1)
  const int8_t *add_src;   // the residual, or null
  int8_t *add_dst;         // the sum, or null
  int8_t *y;               // the projection's result, or null (then the sum is what the caller wants)
  uint32_t x_bytes;
  int ih, iw, x_cs, x_cw, oh, ow;   // x_cw: input channels rounded up to 16
  int ks_in;                        // K slices of the expansion
  int ocw, y_cs;                    // projection channels rounded up to 16, channel stride of y / add_src / add_dst
  int kh, kw, sh, sw, pt, pl, dh, dw;
  int relu_ex, relu_dw, relu_pw;
  int add_m_src, add_m_conv, add_rshift, add_relu, add_pk;
  int rows, width;                   // a pixel block: R rows of W pixels
  int xblocks, rblocks, rgroups;     // column blocks per output row, row blocks per image, groups of P row blocks
  uint32_t magic_w, magic_pc;        // ceil(2^32 / width), ceil(2^32 / pcols)
  int pcols, prows;                  // the patch of a group
  int lp16;                          // LDS pitch of a patch pixel in 16-byte chunks (odd)
  int xc16, xp16;                    // 16-byte chunks of an input pixel, and its LDS pitch in chunks (odd)
  uint32_t magic_xc;                 // ceil(2^32 / xc16)
  int log2p, n_cb, n_tm, ngroups, nk;
};

// NW waves per workgroup; NT result blocks of the projection per wave
template <int NW, int NT>
__global__ __launch_bounds__(NW * 64) __attribute__((amdgpu_waves_per_eu(NW == 16 ? 4 : 3, NW == 16 ? 4 : 3))) void
conv_irb_kernel(IrbArgs a) {
  extern __shared__ __align__(16) uint8_t smem[];
  const int P = 1 << a.log2p;
  const int ocp = a.n_tm * 32;
  const int tiles = a.n_tm << a.log2p;
  v4i *bfr = reinterpret_cast<v4i *>(smem);                                         // [P][n_cb][64 lanes]
  int32_t *q2 = reinterpret_cast<int32_t *>(smem + (size_t)P * a.n_cb * 1024);        // the projection's planes
  int32_t *qall = q2 + 5 * ocp;                                                     // [NW][160]
  int32_t *red = qall + NW * 160;                                                   // [tiles][16][64] when nk > 1
  v4i *patch = reinterpret_cast<v4i *>(red + (a.nk > 1 ? tiles * 1024 : 0));         // [prows * pcols][lp16 chunks]
  v4i *xin = patch + a.prows * a.pcols * a.lp16;                                    // [prows * pcols][xp16 chunks]

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int p32 = lane & 31, fk = lane >> 5;
  // workgroups are dealt to the 8 XCDs round-robin; each XCD takes a contiguous run of groups
  const int per_xcd = (a.ngroups + 7) >> 3;
  const int xcd = (int)(blockIdx.x & 7);
  const int g = xcd * per_xcd + (int)(blockIdx.x >> 3);
  if (g >= a.ngroups || g >= (xcd + 1) * per_xcd) return;   // the whole workgroup: no barrier is missed
  // group -> (image, column block, group of P row blocks)
  const int t0 = g / a.rgroups;
  const int rg = g - t0 * a.rgroups;
  const int n = t0 / a.xblocks;
  const int xb = t0 - n * a.xblocks;
  const int rb0 = rg << a.log2p;
  const int nb = min(P, a.rblocks - rb0);                   // pixel blocks of this group that exist

  for (int i = threadIdx.x; i < 5 * ocp; i += NW * 64) q2[i] = a.qpw[i];
  if (a.nk > 1)
    for (int i = threadIdx.x; i < tiles * 1024; i += NW * 64) red[i] = 0;

  int32_t *qw = qall + wave * 160;
  const int32_t *pc64 = qw + fk * 32, *pmult = qw + 64 + fk * 16, *pshift = qw + 96 + fk * 16, *phpot = qw + 128 + fk * 16;
  auto params_to_lds = [&](const int32_t *src) {
    qw[lane] = src[lane];
    qw[64 + lane] = src[64 + lane];
    if (lane < 32) qw[128 + lane] = src[128 + lane];
  };

  // ---- phase A: expansion into the LDS patch -------------------------------
  {
    const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
    const int row_bytes = a.iw * a.x_cs;
    const uint32_t img_base = (uint32_t)n * (uint32_t)(a.ih * row_bytes);
    const int prow0 = rb0 * a.rows * a.sh - a.pt;             // input row / column of the patch's first pixel
    const int pcol0 = xb * a.width * a.sw - a.pl;
    const int prows = (nb * a.rows - 1) * a.sh + (a.kh - 1) * a.dh + 1;   // rows this group's windows span
    const int npp = prows * a.pcols;
    const int npb = (npp + 31) >> 5;
    // the input pixels under the patch, fetched once by the whole workgroup (one trip to memory instead of
    // one per result block): 16-byte chunks in memory order, zeros outside the image
    {
      const int chunks = npp * a.xc16;
      for (int q0 = 0; q0 < chunks; q0 += 4 * NW * 64) {
        v4i v[4];
        int dst[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (q0 + u * NW * 64 >= chunks) break;              // the same for the whole workgroup
          const int q = q0 + u * NW * 64 + (int)threadIdx.x;
          const int pix = a.xc16 == 1 ? q : (int)__umulhi((uint32_t)q, a.magic_xc), cc = q - pix * a.xc16;
          const int pr = (int)__umulhi((uint32_t)pix, a.magic_pc), pc = pix - pr * a.pcols;
          const int ih = prow0 + pr, iw = pcol0 + pc;
          const bool ok = (q < chunks) & ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
          v[u] = (v4i)__builtin_amdgcn_raw_buffer_load_b128(
              xrsrc, ok ? (uint32_t)(ih * row_bytes + iw * a.x_cs + cc * 16) : kOobOffset, img_base, 0);
          dst[u] = q < chunks ? pix * a.xp16 + cc : -1;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (q0 + u * NW * 64 >= chunks) break;
          if (dst[u] >= 0) xin[dst[u]] = v[u];
        }
      }
    }
    __syncthreads();
    for (int cb = wave; cb < a.n_cb; cb += NW) {
      v4i afr[kIrbMaxKsIn];
      const v4i *afrag = reinterpret_cast<const v4i *>(a.wex) + (size_t)cb * a.ks_in * 64 + lane;
#pragma unroll
      for (int ks = 0; ks < kIrbMaxKsIn; ++ks) afr[ks] = ks < a.ks_in ? afrag[ks * 64] : v4i{0, 0, 0, 0};
      params_to_lds(a.qex + (size_t)cb * 160);
      for (int pb = 0; pb < npb; ++pb) {
        const int pp = pb * 32 + p32;
        const int pr = (int)__umulhi((uint32_t)pp, a.magic_pc), pc = pp - pr * a.pcols;
        const int ih = prow0 + pr, iw = pcol0 + pc;
        const bool valid = (pp < npp) & ((unsigned)ih < (unsigned)a.ih) & ((unsigned)iw < (unsigned)a.iw);
        const v4i *xp = xin + min(pp, npp - 1) * a.xp16 + fk;
        v16i acc[1];
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][e] = 0;
#pragma unroll
        for (int ks = 0; ks < kIrbMaxKsIn; ++ks) {
          if (ks >= a.ks_in) break;                          // the same for the whole wave
          // a K slice past the input's last 16 channels meets zero filter columns: any pixel's chunk will do
          const v4i bx = xp[min(ks * 2, a.xc16 - 1 - fk)];
          acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(afr[ks], bx, acc[0], 0, 0, 0);
        }
        uint32_t outw[1][4];
        if (a.relu_ex) requant_rows_c64<1, true>(acc, 0, pc64, pmult, pshift, phpot, outw);
        else requant_rows_c64<1, false>(acc, -128, pc64, pmult, pshift, phpot, outw);
        // outside the image the depthwise conv sees its padding: zeros, not the expansion of zeros
        const v4i o = valid ? v4i{(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]} : v4i{0, 0, 0, 0};
        if (pp < npp) patch[pp * a.lp16 + cb * 2 + fk] = o;
      }
    }
  }
  __syncthreads();

  // what never changes for a lane: its pixel within a block (lanes past R * W repeat pixel 0 and store nothing)
  const bool in_block = p32 < a.rows * a.width;
  const int lr = in_block ? (int)__umulhi((uint32_t)p32, a.magic_w) : 0;
  const int lc = in_block ? p32 - lr * a.width : 0;
  const int ow = xb * a.width + lc;
  const bool col_ok = in_block & (ow < a.ow);

  // ---- phase B: depthwise, from the patch ----------------------------------
  {
    const int lane_px = ((lr * a.sh) * a.pcols + lc * a.sw) * a.lp16 + fk;
    int tap_off[3][3];                                      // a tap's offset from the window origin, in chunks
#pragma unroll
    for (int i = 0; i < 3; ++i)
#pragma unroll
      for (int j = 0; j < 3; ++j) tap_off[i][j] = (min(i, a.kh - 1) * a.dh * a.pcols + min(j, a.kw - 1) * a.dw) * a.lp16;
    // a lane's dword of a diagonal fragment sits in dword (row >> 3) of its four
    const int dsel = p32 >> 3;
    const int m0 = dsel == 0 ? -1 : 0, m1 = dsel == 1 ? -1 : 0, m2 = dsel == 2 ? -1 : 0, m3 = dsel == 3 ? -1 : 0;
    const int T = a.n_cb * nb;                              // items: (K slice, pixel block), K-slice major
    const int chunk = (T + NW - 1) / NW;
    int it = wave * chunk;
    const int it_end = min(T, it + chunk);
    while (it < it_end) {
      const int cb = it / nb, p0 = it - cb * nb;
      const int p1 = min(nb, p0 + (it_end - it));
      it += p1 - p0;
      int wv[9];
      {
        const uint32_t *wsrc = a.wdw + (size_t)cb * 9 * 64 + lane;
#pragma unroll
        for (int t = 0; t < 9; ++t) wv[t] = (int)wsrc[t * 64];   // taps the window does not have are stored as zeros
        params_to_lds(a.qdw + (size_t)cb * 160);
      }
      for (int p = p0; p < p1; ++p) {
        const v4i *win = patch + (p * a.rows * a.sh * a.pcols) * a.lp16 + lane_px + cb * 2;
        v16i acc[1];
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[0][e] = 0;
#pragma unroll
        for (int i = 0; i < 3; ++i)
#pragma unroll
          for (int j = 0; j < 3; ++j) {
            const int w = wv[i * 3 + j];
            const v4i af = {w & m0, w & m1, w & m2, w & m3};
            acc[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(af, win[tap_off[i][j]], acc[0], 0, 0, 0);
          }
        uint32_t outw[1][4];
        if (a.relu_dw) requant_rows_c64<1, true>(acc, 0, pc64, pmult, pshift, phpot, outw);
        else requant_rows_c64<1, false>(acc, -128, pc64, pmult, pshift, phpot, outw);
        bfr[(p * a.n_cb + cb) * 64 + lane] = v4i{(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
      }
    }
  }
  __syncthreads();

  // ---- phase C: projection --------------------------------------------------
  {
    // a unit of work: (result block t, part kp of its K slices); result block t -> (channel block t >> log2p,
    // pixel block t & (P - 1)).  nk > 1: wave w takes block w % tiles, part w / tiles, and the parts meet in
    // LDS; nk == 1: wave w takes blocks w, w + NW, ...
    int tl[NT], tm[NT], pp[NT];
    bool on[NT];
    const int kp = a.nk > 1 ? wave / tiles : 0;
    const int kper = (a.n_cb + a.nk - 1) / a.nk;
    const int k0 = kp * kper, k1 = min(a.n_cb, k0 + kper);
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      tl[i] = a.nk > 1 ? wave - kp * tiles : wave + NW * i;
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
      const int oh = (rb0 + pp[i]) * a.rows + lr;
      const int oc = tm[i] * 32 + fk * 16;
      const bool st_ok = col_ok & (oh < a.oh) & (oc < a.ocw);
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

struct IrbPlan {
  int rows, width, xblocks, rblocks, rgroups, ngroups;
  int pcols, prows, lp16, ks_in;
  int n_cb, n_tm, log2p, nw, nt, nk;
  unsigned lds;
};

// (waves per workgroup, result blocks per wave) the kernel is built for
constexpr int kIrbShapes[][2] = {{8, 1}, {8, 2}, {8, 3}, {16, 1}, {16, 2}};
const char *const kIrbNames[] = {"mfma_irb_w8_nt1", "mfma_irb_w8_nt2", "mfma_irb_w8_nt3", "mfma_irb_w16_nt1", "mfma_irb_w16_nt2"};
constexpr int kNumIrbShapes = 5;

int irb_shape_index(int nw, int nt) {
  for (int i = 0; i < kNumIrbShapes; ++i)
    if (kIrbShapes[i][0] == nw && kIrbShapes[i][1] == nt) return i;
  return -1;
}

bool irb_plan(const tpuhip_conv_desc &e, const tpuhip_conv_desc &d, const tpuhip_conv_desc &p, IrbPlan *out) {
  if (!is_pointwise_conv(e) || e.ic > 32 * kIrbMaxKsIn || e.ic < 1 || e.x_cs % 16 || e.x_cs < e.ic) return false;
  const bool depthwise = d.g == d.ic && d.g == d.oc && d.g > 1 && !d.ins_h && !d.ins_w && !d.relu_first;
  if (!depthwise || d.kh < 1 || d.kw < 1 || d.kh > 3 || d.kw > 3) return false;
  if (d.n != e.n || d.ih != e.oh || d.iw != e.ow || d.ic != e.oc || d.x_cs != e.y_cs) return false;
  if (!is_pointwise_conv(p) || p.n != d.n || p.ih != d.oh || p.iw != d.ow || p.ic != d.oc || p.x_cs != d.y_cs) return false;
  if (d.x_cs % 16 || d.y_cs % 16 || p.y_cs % 16 || p.y_cs < p.oc) return false;
  if (d.sh < 1 || d.sw < 1 || d.dh < 1 || d.dw < 1 || d.sh > 4 || d.sw > 4 || d.dh > 8 || d.dw > 8 || d.pl > 64 || d.pt > 64)
    return false;
  if ((int64_t)e.n * e.ih * e.iw * e.x_cs >= (1ll << 31) || (int64_t)p.n * p.oh * p.ow * p.y_cs >= (1ll << 31)) return false;
  out->n_cb = (d.oc + 31) / 32;
  out->n_tm = (p.oc + 31) / 32;
  out->ks_in = (e.ic + 31) / 32;
  if (out->n_cb > 64 || out->n_tm > 12) return false;
  out->lp16 = 2 * out->n_cb + 1;
  // block shapes in the order of the blocks they cut an image into (fewest first); the first whose patch fits
  int order[4] = {1, 2, 3, 4};
  auto blocks_of = [&](int rows) { return (int64_t)((d.oh + rows - 1) / rows) * ((d.ow + 32 / rows - 1) / (32 / rows)); };
  std::stable_sort(order, order + 4, [&](int x, int y) { return blocks_of(x) < blocks_of(y); });
  for (int oi = 0; oi < 4; ++oi) {
    const int rows = order[oi], width = 32 / rows;
    const int64_t best = blocks_of(rows);
    if (best * d.n >= (1ll << 28)) continue;
    out->rows = rows; out->width = width;
    out->rblocks = (d.oh + rows - 1) / rows;
    out->xblocks = (d.ow + width - 1) / width;
    out->pcols = (width - 1) * d.sw + (d.kw - 1) * d.dw + 1;
    // pixel blocks per workgroup: two where that still leaves a workgroup per CU and the patch small; waves per
    // workgroup: eight, two workgroups to a CU, while the LDS allows it, else sixteen
    for (int log2p = (best * d.n >= 1024 ? 1 : 0); log2p >= 0; --log2p) {
      const int P = 1 << log2p, tiles = out->n_tm * P;
      const int prows = (P * rows - 1) * d.sh + (d.kh - 1) * d.dh + 1;
      const int xp16 = ((e.ic + 15) / 16) | 1;
      const int64_t patch = (int64_t)prows * out->pcols * (out->lp16 + xp16) * 16;   // the expanded patch and the input under it
      for (int nw = 8; nw <= 16; nw *= 2) {
        const int nt = (tiles + nw - 1) / nw;
        if (irb_shape_index(nw, nt) < 0) continue;
        const int nk = tiles < nw ? std::min(nw / tiles, out->n_cb) : 1;
        const int64_t lds = (int64_t)out->n_cb * P * 1024 + 5 * out->n_tm * 32 * 4 + nw * 160 * 4 + (nk > 1 ? tiles * 4096 : 0) + patch;
        if (lds > (nw == 8 ? 80 : 160) * 1024) continue;
        out->log2p = log2p; out->nw = nw; out->nt = nt; out->nk = nk; out->prows = prows; out->lds = (unsigned)lds;
        out->rgroups = (out->rblocks + P - 1) / P;
        out->ngroups = d.n * out->xblocks * out->rgroups;
        return true;
      }
    }
  }
  return false;
}

// per-channel planes regrouped per 32-channel block: 32 addend pairs | 32 mult | 32 shift | 32 2^(r-1)
std::vector<int32_t> planes_per_block(const std::vector<int32_t> &p, int n_cb) {
  const int cp = n_cb * 32;
  std::vector<int32_t> q((size_t)n_cb * 160, 0);
  for (int cb = 0; cb < n_cb; ++cb)
    for (int i = 0; i < 32; ++i) {
      const int chn = cb * 32 + i;
      int32_t *o = q.data() + (size_t)cb * 160;
      o[2 * i] = p[2 * chn];
      o[2 * i + 1] = p[2 * chn + 1];
      o[64 + i] = p[2 * cp + chn];
      o[96 + i] = p[3 * cp + chn];
      o[128 + i] = p[4 * cp + chn];
    }
  return q;
}

// [32-channel block][9][lane]: the one dword of the lane's diagonal fragment that can be nonzero --
// lane l holds MFMA row l & 31 = channel mfma_row_to_oc(row) of the block and K bytes 16 * (l >> 5) .. + 15;
// the weight sits at byte (channel in block) - 16 * (l >> 5) where that is inside the lane's 16
std::vector<uint32_t> diagonal_dwords(const int8_t *filter, int c, int n_cb, int kh, int kw) {
  std::vector<uint32_t> out((size_t)n_cb * 9 * 64, 0);
  for (int cb = 0; cb < n_cb; ++cb)
    for (int i = 0; i < kh; ++i)
      for (int j = 0; j < kw; ++j)
        for (int lane = 0; lane < 64; ++lane) {
          const int row = lane & 31;
          const int ch_in_block = mfma_row_to_oc(row, 1);
          const int ch = cb * 32 + ch_in_block;
          const int b = ch_in_block - 16 * (lane >> 5);
          if (ch >= c || b < 0 || b >= 16 || (b >> 2) != (row >> 3)) continue;
          out[((size_t)cb * 9 + i * 3 + j) * 64 + lane] = (uint32_t)(uint8_t)filter[((size_t)ch * kh + i) * kw + j] << (8 * (b & 3));
        }
  return out;
}

}  // namespace

namespace tpuhip {

const char *irb_variant_name(int i) { return i >= 0 && i < kNumIrbShapes ? kIrbNames[i] : nullptr; }

bool irb_covers(const tpuhip_conv_desc &e, const tpuhip_conv_desc &d, const tpuhip_conv_desc &p) {
  IrbPlan plan;
  return irb_plan(e, d, p, &plan);
}

int irb_prepack(tpuhip_ctx *ctx, tpuhip_conv_chain *ch, const tpuhip_chain_conv *ce, const tpuhip_chain_conv *cd,
                const tpuhip_chain_conv *cp) {
  const tpuhip_conv_desc &e = ch->da, &d = ch->db, &p = ch->dc;
  IrbPlan plan;
  if (!irb_plan(e, d, p, &plan)) return set_error(TPUHIP_ERR_UNSUPPORTED, "conv chain: shapes not covered");
  // every diagonal dword must land where the kernel looks for it
  for (int row = 0; row < 32; ++row) {
    const int chb = mfma_row_to_oc(row, 1);
    const int b = chb - 16 * ((row >> 2) & 1);
    if (b < 0 || b >= 16 || (b >> 2) != (row >> 3)) return set_error(TPUHIP_ERR_INVALID, "conv chain: fragment layout");
  }
  std::vector<int32_t> pe, pd, pp;
  const int cp_ = plan.n_cb * 32, ocp = plan.n_tm * 32;
  if (!requant_planes(e.oc, cp_, (size_t)e.ic, e.do_relu != 0, ce->filter, (e.with_bias && ce->bias) ? ce->bias : nullptr,
                      ce->multiplier, ce->rshift, &pe) ||
      !requant_planes(d.oc, cp_, (size_t)d.kh * d.kw, d.do_relu != 0, cd->filter, (d.with_bias && cd->bias) ? cd->bias : nullptr,
                      cd->multiplier, cd->rshift, &pd) ||
      !requant_planes(p.oc, ocp, (size_t)p.ic, p.do_relu != 0, cp->filter, (p.with_bias && cp->bias) ? cp->bias : nullptr,
                      cp->multiplier, cp->rshift, &pp))
    return set_error(TPUHIP_ERR_UNSUPPORTED,
                     "conv chain: needs right shifts of at least 1 and sums that cannot overflow the rounding");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const std::vector<int8_t> fe = mfma_a_fragments(ce->filter, e.oc, plan.n_cb, e.ic, plan.ks_in * 32, 1);
  const std::vector<uint32_t> fd = diagonal_dwords(cd->filter, d.oc, plan.n_cb, d.kh, d.kw);
  const std::vector<int8_t> fp = mfma_a_fragments(cp->filter, p.oc, plan.n_tm, p.ic, cp_, 1);
  int rc = upload_vec(ctx, fe, &ch->w1);
  if (!rc) rc = upload_vec(ctx, fd, &ch->w2d);
  if (!rc) rc = upload_vec(ctx, fp, &ch->w3);
  if (!rc) rc = upload_vec(ctx, planes_per_block(pe, plan.n_cb), &ch->q1);
  if (!rc) rc = upload_vec(ctx, planes_per_block(pd, plan.n_cb), &ch->q2);
  if (!rc) rc = upload_vec(ctx, pp, &ch->q3);
  ch->variant = irb_shape_index(plan.nw, plan.nt);
  ch->name = kIrbNames[ch->variant];
  return rc;
}

int irb_run(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y, const tpuhip_conv_post *post) {
  const tpuhip_conv_desc &e = ch->da, &d = ch->db, &p = ch->dc;
  IrbPlan plan;
  TPUHIP_REQUIRE(irb_plan(e, d, p, &plan), "conv chain: shapes not covered");
  TPUHIP_REQUIRE(!(post && (post->lut || post->pool)), "conv chain: an inverted-residual chain takes an add behind its last conv and nothing else");
  const bool add = post && post->add.enable;
  TPUHIP_REQUIRE(!add || (post->add_src && post->add_out), "conv chain: fused add without its operand or result");
  TPUHIP_REQUIRE(y || add, "conv chain: nothing to write");
  IrbArgs a{};
  a.x = (const int8_t *)x;
  a.wex = ch->w1; a.qex = ch->q1;
  a.wdw = ch->w2d; a.qdw = ch->q2;
  a.wpw = ch->w3; a.qpw = ch->q3;
  a.y = (int8_t *)y;
  if (add) {
    const tpuhip_fused_add &f = post->add;
    TPUHIP_REQUIRE(f.rshift >= 0 && f.rshift <= 30, "conv chain: add rshift %d outside [0,30]", f.rshift);
    TPUHIP_REQUIRE(f.m_src >= -128 && f.m_src <= 127 && f.m_conv >= -128 && f.m_conv <= 127,
                   "conv chain: add multipliers must be int8");
    a.add_src = (const int8_t *)post->add_src;
    a.add_dst = (int8_t *)post->add_out;
    a.add_m_src = f.m_src;
    a.add_m_conv = f.m_conv;
    a.add_rshift = f.rshift;
    a.add_relu = f.do_relu ? 1 : 0;
    a.add_pk = std::abs(f.m_src) <= 127 && std::abs(f.m_conv) <= 127 && f.rshift <= 8;
  }
  a.x_bytes = (uint32_t)((int64_t)e.n * e.ih * e.iw * e.x_cs);
  a.ih = e.ih; a.iw = e.iw; a.x_cs = e.x_cs; a.x_cw = (e.ic + 15) / 16 * 16; a.oh = d.oh; a.ow = d.ow;
  a.ks_in = plan.ks_in;
  a.ocw = (p.oc + 15) / 16 * 16; a.y_cs = p.y_cs;
  a.kh = d.kh; a.kw = d.kw; a.sh = d.sh; a.sw = d.sw; a.pt = d.pt; a.pl = d.pl; a.dh = d.dh; a.dw = d.dw;
  a.relu_ex = e.do_relu ? 1 : 0;
  a.relu_dw = d.do_relu ? 1 : 0;
  a.relu_pw = p.do_relu ? 1 : 0;
  auto magic = [](int dv) { return dv > 1 ? (uint32_t)(((1ull << 32) + dv - 1) / (uint64_t)dv) : 0u; };
  a.rows = plan.rows; a.width = plan.width;
  a.xblocks = plan.xblocks; a.rblocks = plan.rblocks; a.rgroups = plan.rgroups;
  a.magic_w = magic(plan.width);
  a.pcols = plan.pcols; a.prows = plan.prows;
  a.magic_pc = magic(plan.pcols);
  a.lp16 = plan.lp16;
  a.xc16 = a.x_cw / 16;
  a.xp16 = a.xc16 | 1;
  a.magic_xc = magic(a.xc16);
  a.log2p = plan.log2p; a.n_cb = plan.n_cb; a.n_tm = plan.n_tm; a.ngroups = plan.ngroups; a.nk = plan.nk;
  const unsigned lds = plan.lds;
  const dim3 grid(8u * (unsigned)((a.ngroups + 7) / 8)), block((unsigned)plan.nw * 64);
#define TPUHIP_IRB_LAUNCH(NWV, NTV)                                                                       \
  if (plan.nw == NWV && plan.nt == NTV) {                                                                 \
    auto kernel = conv_irb_kernel<NWV, NTV>;                                                              \
    TPUHIP_REQUIRE(raise_dynamic_lds((const void *)kernel, lds), "conv chain: raising the LDS limit failed"); \
    if (ctx->prof_start)                                                                                  \
      hipExtLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                  \
      hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, a);                                       \
  }
  TPUHIP_IRB_LAUNCH(8, 1)
  TPUHIP_IRB_LAUNCH(8, 2)
  TPUHIP_IRB_LAUNCH(8, 3)
  TPUHIP_IRB_LAUNCH(16, 1)
  TPUHIP_IRB_LAUNCH(16, 2)
#undef TPUHIP_IRB_LAUNCH
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // namespace tpuhip

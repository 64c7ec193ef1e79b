// Two pointwise convolutions as one launch: conv A (1x1, at most 128 input channels, 256 or 512
// output channels, optionally with an EltwiseAdd folded behind it) and conv B (1x1) that reads
// what A -- or the add -- produced.  In a residual network this is the 1x1 expansion + add at the
// end of one bottleneck block followed by the 1x1 reduction that opens the next: the sum is
// written once and never read back, and one launch disappears.
//
//   Conv2DOpKernel::invoke (core/conv.cpp:80-104) for A, EltwiseAddOpKernel::i8_invoke
//   (core/eltwise.cpp:52-85) on (add_src, A's result), Conv2DOpKernel::invoke for B -- the same
//   bytes as the three run one after the other.
//
// A workgroup of eight waves owns a tile of BN pixels and ALL output channels of both convs:
//   * the filters never touch LDS: a wave's share of A's filter (OC1 / 8 channels x K) and B's
//     (one 32-channel block x OC1) are MFMA A-operand fragments held in registers for the
//     lifetime of the workgroup, loaded once from global memory in fragment order;
//   * a tile's pixels (BN rows of K bytes) are fetched two tiles ahead into registers and
//     parked, one tile ahead, in a double-buffered LDS tile;
//   * GEMM 1: every wave multiplies its channels by the whole pixel tile, requantises into the
//     staged tile [pixel][OC1 + 16 bytes] in LDS;
//   * flush: threads walk the staged tile in memory order (whole rows of the tensors): store of
//     A's result where the caller keeps it, the add with its other operand (requested before
//     GEMM 1), store of the sum, and the sum written back over the staged tile;
//   * GEMM 2: the staged tile is exactly B's MFMA operand (pixel rows of OC1 bytes); the
//     32x32 blocks of B's result are dealt to the waves, requantised from the registers and
//     stored 16 bytes per lane.
// Two barriers per tile; the staged tile is double-buffered so that GEMM 2 of one tile and the
// requantisation of the next overlap.
#include "conv_chain.hpp"

#include <cstring>

using namespace tpuhip;

struct ChainArgs {
  const int8_t *x;         // conv A's input, [npix][x_cs]
  const int8_t *w1;        // A fragments of conv A: [wave][32-channel block][K slice][lane][16]
  const int8_t *w2;        // A fragments of conv B: [32-channel block][K slice][lane][16]
  const int32_t *q1;       // conv A per channel: (low, high) pairs of the 64-bit addend | multiplier | shift | 2^(r-1)
  const int32_t *q2;       // conv B likewise
  int8_t *y_a;             // conv A's own result, or null
  const int8_t *add_src;   // the add's other operand, or null: B reads A's result
  int8_t *add_dst;         // the sum, or null
  int8_t *y_b;
  int npix, x_cs;
  int n_tiles, n_full;     // tiles in all; the first n_full hold BN pixels, the rest 32
  uint32_t x_bytes;
  int lo1, lo2;            // 0: the conv clamps at 0 (ReLU) and its planes hold the short form
  int add_m_src, add_m_conv, add_rshift, add_relu, add_pk;
#ifdef TPUHIP_TRACE
  unsigned long long *trace;   // development builds: 32 shader-clock stamps per wave
#endif
};
#ifdef TPUHIP_TRACE
#define CHAIN_TS(k) (ts[k] = (unsigned long long)clock64())
#else
#define CHAIN_TS(k) ((void)0)
#endif

// W2LDS: conv B's filter fragments sit in LDS instead of registers (registers are what limits
// the workgroups per CU of the narrow variant)
template <int OC1, int KP1, int OC2, int BN, bool W2LDS>
constexpr unsigned chain_lds_bytes() {
  return 2u * BN * KP1 + 2u * BN * (OC1 + 16) + 20u * OC1 + 20u * OC2 + (W2LDS ? OC1 * OC2 : 0);
}

template <int OC1, int KP1, int OC2, int BN, int OCC, bool W2LDS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(OCC, OCC))) void conv_chain_kernel(ChainArgs a) {
#ifdef TPUHIP_TRACE
  unsigned long long ts[32] = {};
  int nt = 0;
#endif
  CHAIN_TS(0);
  constexpr int NT = 512, NW = 8;
  constexpr int TM1 = OC1 / NW / 32;      // 32-channel blocks of conv A per wave
  constexpr int TN = BN / 32;             // 32-pixel blocks of a tile
  constexpr int KS1 = KP1 / 32;           // 32-byte K slices of GEMM 1
  constexpr int KC1 = KP1 / 64;
  constexpr int SROW = OC1 + 16;          // bytes of a staged pixel row
  constexpr int KS2 = OC1 / 32;           // K slices of GEMM 2
  constexpr int NB2 = (OC2 / 32) * TN;    // 32x32 blocks of conv B's tile
  constexpr int CPRK = KP1 / 16;          // 16-byte chunks of an input pixel row
  constexpr int XCH = BN * CPRK;          // ... of an input tile
  constexpr int CPR = OC1 / 16;           // chunks of a staged row
  constexpr int NU = BN * CPR / NT;       // staged chunks per thread
  static_assert(TM1 >= 1 && TM1 * NW * 32 == OC1 && TN >= 1 && TN * 32 == BN, "bad tile");
  static_assert(NB2 >= 1 && NB2 <= NW && XCH <= NT && NU * NT == BN * CPR && KC1 * 64 == KP1, "bad tile");
  static_assert(TN <= 2 && NU % TN == 0 && NT % CPR == 0 && (NU / TN) * (NT / CPR) == 32, "chunk walk: the first NU / TN chunks are the first 32 rows");
  extern __shared__ __attribute__((aligned(16))) v4i chain_smem[];
  v4i *const xB = chain_smem;                                                  // [2][KC1][BN][4 chunks], swizzled
  int8_t *const stage0 = reinterpret_cast<int8_t *>(xB + 2 * KC1 * BN * 4);    // [2][BN][SROW]
  int32_t *const q1 = reinterpret_cast<int32_t *>(stage0 + 2 * BN * SROW);     // 5 planes of OC1
  int32_t *const q2 = q1 + 5 * OC1;                                            // 5 planes of OC2
  v4i *const w2l = reinterpret_cast<v4i *>(q2 + 5 * OC2);                      // W2LDS: [block][K slice][lane]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int frow = lane & 31, fk = lane >> 5;
  int tile = blockIdx.x;
  if (tile >= a.n_tiles) return;
  const int tstep = gridDim.x;

  // Tiles of the launch: n_full tiles of BN pixels, then (TN == 2) tiles of 32 pixels for what is left,
  // so that the last round of the workgroups' walk costs half a round where it is not full.
  // Every tensor is addressed through a buffer descriptor with 32-bit offsets: a pixel past the
  // end reads zeros and its stores are dropped, no branch and no 64-bit arithmetic per access.
  const __amdgpu_buffer_rsrc_t xrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.x, 0, a.x_bytes, 0x00020000);
  const uint32_t big_bytes = (uint32_t)a.npix * (uint32_t)OC1;
  const __amdgpu_buffer_rsrc_t srsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.add_src, 0, a.add_src ? big_bytes : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t zrsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.add_dst, 0, a.add_dst ? big_bytes : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t yarsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a.y_a, 0, a.y_a ? big_bytes : 0, 0x00020000);
  const __amdgpu_buffer_rsrc_t ybrsrc =
      __builtin_amdgcn_make_buffer_rsrc((void *)a.y_b, 0, (uint32_t)a.npix * (uint32_t)OC2, 0x00020000);
  auto tile_pix0 = [&](int t) { return t < a.n_full ? t * BN : a.n_full * BN + (t - a.n_full) * 32; };
  auto tile_blocks = [&](int t) { return t < a.n_full ? TN : 1; };

  const int lc = tid % CPRK, lrow = tid / CPRK;
  const bool loader = XCH == NT || tid < XCH;
  v4i breg;
  auto load_B = [&](int t) {
    const bool ok = loader && t < a.n_tiles && lrow < 32 * tile_blocks(t);
    breg = buffer_load16(xrsrc, ok ? (uint32_t)((tile_pix0(t) + lrow) * a.x_cs + lc * 16) : kOobOffset);
  };
  auto store_B = [&](int slot) {
    if (loader) xB[slot * (KC1 * BN * 4) + (lc >> 2) * (BN * 4) + lrow * 4 + ((lc & 3) ^ ((lrow >> 2) & 3))] = breg;
  };

  load_B(tile);
  // the filters: this wave's fragments, for the lifetime of the workgroup
  v4i fa1[TM1][KS1];
#pragma unroll
  for (int i = 0; i < TM1; ++i)
#pragma unroll
    for (int ks = 0; ks < KS1; ++ks)
      fa1[i][ks] = reinterpret_cast<const v4i *>(a.w1)[((wave * TM1 + i) * KS1 + ks) * 64 + lane];
  const int ob = wave / TN, pb = wave % TN;   // conv B: this wave's block of the tile
  v4i fa2[W2LDS ? 1 : KS2];
  if (!W2LDS && wave < NB2) {
#pragma unroll
    for (int ks = 0; ks < KS2; ++ks) fa2[ks] = reinterpret_cast<const v4i *>(a.w2)[(ob * KS2 + ks) * 64 + lane];
  }
  // What goes to LDS once -- the parameter planes, conv B's filter (W2LDS) -- is requested in one
  // go and parked afterwards: one trip to memory for all of it, not one per piece.
  constexpr int NQ1 = (5 * OC1 / 4 + NT - 1) / NT, NQ2 = (5 * OC2 / 4 + NT - 1) / NT;
  constexpr int NW2 = W2LDS ? (OC1 * OC2 / 16 + NT - 1) / NT : 0;
  v4i rq1[NQ1], rq2[NQ2], rw2[NW2 > 0 ? NW2 : 1];
#pragma unroll
  for (int u = 0; u < NQ1; ++u)
    if (tid + u * NT < 5 * OC1 / 4) rq1[u] = reinterpret_cast<const v4i *>(a.q1)[tid + u * NT];
#pragma unroll
  for (int u = 0; u < NQ2; ++u)
    if (tid + u * NT < 5 * OC2 / 4) rq2[u] = reinterpret_cast<const v4i *>(a.q2)[tid + u * NT];
#pragma unroll
  for (int u = 0; u < NW2; ++u)
    if (tid + u * NT < OC1 * OC2 / 16) rw2[u] = reinterpret_cast<const v4i *>(a.w2)[tid + u * NT];
  __builtin_amdgcn_sched_barrier(0);
  auto park_constants = [&]() {
#pragma unroll
    for (int u = 0; u < NQ1; ++u)
      if (tid + u * NT < 5 * OC1 / 4) reinterpret_cast<v4i *>(q1)[tid + u * NT] = rq1[u];
#pragma unroll
    for (int u = 0; u < NQ2; ++u)
      if (tid + u * NT < 5 * OC2 / 4) reinterpret_cast<v4i *>(q2)[tid + u * NT] = rq2[u];
#pragma unroll
    for (int u = 0; u < NW2; ++u)
      if (tid + u * NT < OC1 * OC2 / 16) w2l[tid + u * NT] = rw2[u];
  };
  park_constants();
  store_B(0);
  load_B(tile + tstep);
  __syncthreads();
  CHAIN_TS(1);

  // this thread's chunks of a staged tile: chunk u is (row frow_u, 16-byte column fcc) -- rows in
  // steps of NT / CPR, so that the first NU / TN chunks cover the first 32 rows
  const int frow0 = tid / CPR, fcc = tid % CPR;
  const uint32_t foff0 = (uint32_t)(frow0 * OC1 + fcc * 16);
  int cur = 0;
  for (;;) {
    const int pix0 = tile_pix0(tile);
    const int tn = tile_blocks(tile);          // 32-pixel blocks of this tile (uniform)
    const uint32_t tile_off = (uint32_t)pix0 * (uint32_t)OC1;
#ifdef TPUHIP_TRACE
    const bool tr = nt < 4;
    if (tr) CHAIN_TS(2 + nt * 6);
#endif
    // the add's other operand for this thread's chunks of the tile: asked for now, used after GEMM 1
    v4i sv[NU];
    if (a.add_src) {
#pragma unroll
      for (int u = 0; u < NU; ++u)
        if (u < NU / TN || tn == TN)
          sv[u] = buffer_load16(srsrc, tile_off + foff0 + (uint32_t)(u * (NT / CPR) * OC1));
    }
    // ---- GEMM 1: this wave's channels x the tile's pixels
    v16i acc[TM1][TN];
#pragma unroll
    for (int i = 0; i < TM1; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0;
    const v4i *xb = xB + cur * (KC1 * BN * 4);
#pragma unroll
    for (int ks = 0; ks < KS1; ++ks) {
      v4i fb[TN];
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int r = j * 32 + frow;
        fb[j] = xb[(ks >> 1) * (BN * 4) + r * 4 + ((((ks & 1) << 1) + fk) ^ ((r >> 2) & 3))];
      }
#pragma unroll
      for (int i = 0; i < TM1; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          if (j < tn) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa1[i][ks], fb[j], acc[i][j], 0, 0, 0);
    }
#ifdef TPUHIP_TRACE
    if (tr) CHAIN_TS(3 + nt * 6);
#endif
    // the next tile's pixels go to the other LDS tile, the one after that is requested
    const int next = tile + tstep;
    store_B(cur ^ 1);
    load_B(next + tstep);

    // ---- requantisation of conv A into the staged tile
    int8_t *const stage = stage0 + cur * (BN * SROW);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (j < tn) {
#pragma unroll
        for (int i = 0; i < TM1; ++i) {
          uint32_t outw[1][4];
          const int cb = wave * (32 * TM1) + fk * (16 * TM1) + i * 16;   // the lane's 16 channels of block i
          const v16i (&blk)[1] = reinterpret_cast<const v16i (&)[1]>(acc[i][j]);
          if (a.lo1 == 0)
            requant_rows_c64<1, true>(blk, 0, q1 + 2 * cb, q1 + 2 * OC1 + cb, q1 + 3 * OC1 + cb, q1 + 4 * OC1 + cb, outw);
          else
            requant_rows_c64<1, false>(blk, -128, q1 + 2 * cb, q1 + 2 * OC1 + cb, q1 + 3 * OC1 + cb, q1 + 4 * OC1 + cb, outw);
          *reinterpret_cast<v4i *>(stage + (j * 32 + frow) * SROW + cb) =
              v4i{(int)outw[0][0], (int)outw[0][1], (int)outw[0][2], (int)outw[0][3]};
        }
      }
    }
#ifdef TPUHIP_TRACE
    if (tr) CHAIN_TS(4 + nt * 6);
#endif
    __syncthreads();
#ifdef TPUHIP_TRACE
    if (tr) CHAIN_TS(5 + nt * 6);
#endif

    // ---- flush in memory order: A's result, the add, the sum back into the staged tile
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      if (u < NU / TN || tn == TN) {
        const int row = frow0 + u * (NT / CPR);
        const uint32_t off = tile_off + foff0 + (uint32_t)(u * (NT / CPR) * OC1);
        v4i *const sp = reinterpret_cast<v4i *>(stage + row * SROW + fcc * 16);
        const v4i o = *sp;
        if (a.y_a) __builtin_amdgcn_raw_buffer_store_b128((v4u)o, yarsrc, off, 0, 0);
        if (a.add_src) {
          const v4i z = fused_add_chunk(o, sv[u], a.add_m_src, a.add_m_conv, a.add_rshift, a.add_relu, a.add_pk);
          if (a.add_dst) __builtin_amdgcn_raw_buffer_store_b128((v4u)z, zrsrc, off, 0, 0);
          *sp = z;
        }
      }
    }
#ifdef TPUHIP_TRACE
    if (tr) CHAIN_TS(6 + nt * 6);
#endif
    __syncthreads();
#ifdef TPUHIP_TRACE
    if (tr) CHAIN_TS(7 + nt * 6);
#endif

    // ---- GEMM 2: conv B on the staged tile
    if (wave < NB2 && pb < tn) {
      v16i acc2[1];
#pragma unroll
      for (int e = 0; e < 16; ++e) acc2[0][e] = 0;
      const int8_t *const brow = stage + (pb * 32 + frow) * SROW + fk * 16;
#pragma unroll
      for (int ks = 0; ks < KS2; ++ks)
        acc2[0] = __builtin_amdgcn_mfma_i32_32x32x32_i8(W2LDS ? w2l[(ob * KS2 + ks) * 64 + lane] : fa2[W2LDS ? 0 : ks],
                                                        *reinterpret_cast<const v4i *>(brow + ks * 32), acc2[0], 0, 0, 0);
      uint32_t outw[1][4];
      const int cb = ob * 32 + fk * 16;
      if (a.lo2 == 0)
        requant_rows_c64<1, true>(acc2, 0, q2 + 2 * cb, q2 + 2 * OC2 + cb, q2 + 3 * OC2 + cb, q2 + 4 * OC2 + cb, outw);
      else
        requant_rows_c64<1, false>(acc2, -128, q2 + 2 * cb, q2 + 2 * OC2 + cb, q2 + 3 * OC2 + cb, q2 + 4 * OC2 + cb, outw);
      const v4u o2 = {outw[0][0], outw[0][1], outw[0][2], outw[0][3]};
      __builtin_amdgcn_raw_buffer_store_b128(o2, ybrsrc, (uint32_t)((pix0 + pb * 32 + frow) * OC2 + cb), 0, 0);
    }
#ifdef TPUHIP_TRACE
    ++nt;
#endif
    if (next >= a.n_tiles) break;
    tile = next;
    cur ^= 1;
  }
  CHAIN_TS(30);
#ifdef TPUHIP_TRACE
  ts[31] = (unsigned long long)nt;
  if (a.trace && lane == 0)
    for (int k = 0; k < 32; ++k) a.trace[((size_t)blockIdx.x * 8 + wave) * 32 + k] = ts[k];
#endif
}

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
namespace {

struct ChainVariant {
  int oc1, kp1, oc2, bn, occ;
  const char *name;
};
// X(index, OC1, KP1, OC2, BN, waves per SIMD, conv B's filter in LDS)
#define TPUHIP_CHAIN_VARIANTS(X)     \
  X(0, 256, 64, 64, 64, 4, true)     \
  X(1, 512, 128, 128, 64, 2, false)
const ChainVariant kChainVariants[] = {
#define X(i, OC1, KP1, OC2, BN, O, L) {OC1, KP1, OC2, BN, O, "mfma_chain_" #OC1 "x" #BN "_k" #KP1 "_to" #OC2},
    TPUHIP_CHAIN_VARIANTS(X)
#undef X
};
constexpr int kNumChainVariants = (int)(sizeof(kChainVariants) / sizeof(kChainVariants[0]));

int chain_variant_for(const tpuhip_conv_desc &a, const tpuhip_conv_desc &b) {
  if (!is_pointwise_conv(a) || !is_pointwise_conv(b)) return -1;
  if (a.n != b.n || a.oh != b.ih || a.ow != b.iw || b.ic != a.oc) return -1;
  for (int v = 0; v < kNumChainVariants; ++v) {
    const ChainVariant &c = kChainVariants[v];
    if (a.oc == c.oc1 && a.y_cs == c.oc1 && b.x_cs == c.oc1 && b.oc == c.oc2 && b.y_cs == c.oc2 && a.ic <= c.kp1 &&
        a.ic > c.kp1 / 2 && a.x_cs <= c.kp1 && a.x_cs % 16 == 0 && a.ic > 4 &&
        (int64_t)a.n * a.oh * a.ow * c.oc1 < (1ll << 31))
      return v;
  }
  return -1;
}

bool chain_planes(const tpuhip_conv_desc &d, const int8_t *filter, const int32_t *bias, const int32_t *mult,
                  const int32_t *rshift, std::vector<int32_t> *out) {
  return requant_planes(d.oc, d.oc, (size_t)d.ic, d.do_relu != 0, filter, (d.with_bias && bias) ? bias : nullptr, mult,
                        rshift, out);
}

}  // namespace

extern "C" {

int tpuhip_conv2d_chain_kind(const tpuhip_conv_desc *da, const tpuhip_conv_desc *db) {
  if (!da || !db) return 0;
  if (chain_variant_for(*da, *db) >= 0) return 1;
  return dwpw_covers(*da, *db) ? 2 : 0;
}

int tpuhip_conv2d_can_chain(const tpuhip_conv_desc *da, const tpuhip_conv_desc *db) {
  return tpuhip_conv2d_chain_kind(da, db) != 0 ? 1 : 0;
}

int tpuhip_conv2d_chain_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *da, const tpuhip_conv_desc *db,
                                const int8_t *filter_a, const int32_t *bias_a, const int32_t *mult_a,
                                const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                                const int32_t *mult_b, const int32_t *rshift_b, tpuhip_conv_chain **out) {
  TPUHIP_REQUIRE(ctx && da && db && filter_a && filter_b && mult_a && mult_b && rshift_a && rshift_b && out,
                 "tpuhip_conv2d_chain_prepack: NULL argument");
  const int v = chain_variant_for(*da, *db);
  if (v < 0 && dwpw_covers(*da, *db)) {
    auto *ch = new tpuhip_conv_chain();
    ch->da = *da;
    ch->db = *db;
    ch->kind = 2;
    const int rc = dwpw_prepack(ctx, ch, filter_a, bias_a, mult_a, rshift_a, filter_b, bias_b, mult_b, rshift_b);
    if (rc) {
      tpuhip_conv2d_chain_destroy(ctx, ch);
      return rc;
    }
    *out = ch;
    return TPUHIP_OK;
  }
  if (v < 0)
    return set_error(TPUHIP_ERR_UNSUPPORTED,
                     "conv chain: needs two unpadded 1x1 / stride 1 convs, the first 33..64 -> 256 or 65..128 -> 512 "
                     "channels, the second 256 -> 64 or 512 -> 128, dense channel strides -- or a depthwise conv of "
                     "at most 3 x 3 taps and the unpadded 1x1 / stride 1 conv of at most 384 channels behind it");
  std::vector<int32_t> p1, p2;
  if (!chain_planes(*da, filter_a, bias_a, mult_a, rshift_a, &p1) ||
      !chain_planes(*db, filter_b, bias_b, mult_b, rshift_b, &p2))
    return set_error(TPUHIP_ERR_UNSUPPORTED,
                     "conv chain: needs right shifts of at least 1 and sums that cannot overflow the rounding");
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  const ChainVariant &c = kChainVariants[v];
  auto *ch = new tpuhip_conv_chain();
  ch->da = *da;
  ch->db = *db;
  ch->kind = 1;
  ch->variant = v;
  ch->kp1 = c.kp1;
  ch->name = c.name;
  const std::vector<int8_t> f1 = mfma_a_fragments(filter_a, c.oc1, c.oc1 / 32, da->ic, c.kp1, c.oc1 / 8 / 32);
  const std::vector<int8_t> f2 = mfma_a_fragments(filter_b, c.oc2, c.oc2 / 32, db->ic, c.oc1, 1);
  int rc = upload_vec(ctx, f1, &ch->w1);
  if (!rc) rc = upload_vec(ctx, f2, &ch->w2);
  if (!rc) rc = upload_vec(ctx, p1, &ch->q1);
  if (!rc) rc = upload_vec(ctx, p2, &ch->q2);
  if (rc) {
    tpuhip_conv2d_chain_destroy(ctx, ch);
    return rc;
  }
  *out = ch;
  return TPUHIP_OK;
}

int tpuhip_conv2d_can_chain3(const tpuhip_conv_desc *de, const tpuhip_conv_desc *dd, const tpuhip_conv_desc *dp) {
  return de && dd && dp && irb_covers(*de, *dd, *dp) ? 1 : 0;
}

int tpuhip_conv2d_chain3_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *de, const tpuhip_conv_desc *dd,
                                 const tpuhip_conv_desc *dp, const tpuhip_chain_conv *ce, const tpuhip_chain_conv *cd,
                                 const tpuhip_chain_conv *cp, tpuhip_conv_chain **out) {
  TPUHIP_REQUIRE(ctx && de && dd && dp && ce && cd && cp && out, "tpuhip_conv2d_chain3_prepack: NULL argument");
  TPUHIP_REQUIRE(ce->filter && cd->filter && cp->filter && ce->multiplier && cd->multiplier && cp->multiplier &&
                     ce->rshift && cd->rshift && cp->rshift,
                 "tpuhip_conv2d_chain3_prepack: NULL operand");
  if (!irb_covers(*de, *dd, *dp))
    return set_error(TPUHIP_ERR_UNSUPPORTED,
                     "conv chain: needs an unpadded 1x1 / stride 1 conv of at most 160 input channels, a depthwise conv "
                     "of at most 3 x 3 taps on its result and an unpadded 1x1 / stride 1 conv of at most 384 channels "
                     "on that one's, dense channel strides, and LDS for a pixel block's window of the expanded tensor");
  auto *ch = new tpuhip_conv_chain();
  ch->da = *de;
  ch->db = *dd;
  ch->dc = *dp;
  ch->kind = 3;
  const int rc = irb_prepack(ctx, ch, ce, cd, cp);
  if (rc) {
    tpuhip_conv2d_chain_destroy(ctx, ch);
    return rc;
  }
  *out = ch;
  return TPUHIP_OK;
}

int tpuhip_conv2d_chain3_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y,
                            const tpuhip_conv_post *post) {
  TPUHIP_REQUIRE(ctx && ch && x, "tpuhip_conv2d_chain3_i8: NULL argument");
  TPUHIP_REQUIRE(ch->kind == 3, "tpuhip_conv2d_chain3_i8: not a chain of three");
  return irb_run(ctx, ch, x, y, post);
}

int tpuhip_conv2d_chain_destroy(tpuhip_ctx *ctx, tpuhip_conv_chain *ch) {
  if (!ch) return TPUHIP_OK;
  TPUHIP_REQUIRE(ctx, "tpuhip_conv2d_chain_destroy: NULL context");
  int rc = 0;
  for (void *p : {(void *)ch->w1, (void *)ch->w2, (void *)ch->w3, (void *)ch->w2d, (void *)ch->q1, (void *)ch->q2, (void *)ch->q3}) {
    const int r = p ? tpuhip_free(ctx, p) : 0;
    if (!rc) rc = r;
  }
  delete ch;
  return rc;
}

const char *tpuhip_conv2d_chain_name(const tpuhip_conv_chain *ch) { return ch ? ch->name.c_str() : "null"; }

const char *tpuhip_conv2d_chain_variant_name(int variant) {
  if (variant < 0) return nullptr;
  if (variant < kNumChainVariants) return kChainVariants[variant].name;
  if (const char *n = dwpw_variant_name(variant - kNumChainVariants)) return n;
  return irb_variant_name(variant - kNumChainVariants - 6);
}

int tpuhip_conv2d_chain_post_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y_a,
                                const tpuhip_conv_post *post_a, void *y_b, const tpuhip_conv_post *post_b) {
  TPUHIP_REQUIRE(ctx && ch && x, "tpuhip_conv2d_chain_post_i8: NULL argument");
  TPUHIP_REQUIRE(ch->kind != 3, "conv chain: a chain of three runs through tpuhip_conv2d_chain3_i8");
  TPUHIP_REQUIRE(!(post_a && post_a->pool) && !(post_b && post_b->pool), "conv chain: takes no fused pool");
  if (ch->kind == 2) return dwpw_run(ctx, ch, x, y_a, post_a, y_b, post_b);
  TPUHIP_REQUIRE(!(post_a && post_a->lut) && !(post_b && (post_b->lut || post_b->add.enable)),
                 "conv chain: two pointwise convs take an add behind the first conv and nothing else");
  return tpuhip_conv2d_chain_i8(ctx, ch, x, y_a, post_a ? post_a->add_src : nullptr, post_a ? post_a->add_out : nullptr,
                                post_a ? &post_a->add : nullptr, y_b);
}

int tpuhip_conv2d_chain_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y_a,
                           const void *add_src, void *add_out, const tpuhip_fused_add *f, void *y_b) {
  TPUHIP_REQUIRE(ctx && ch && x && y_b, "tpuhip_conv2d_chain_i8: NULL argument");
  TPUHIP_REQUIRE(ch->kind != 3, "conv chain: a chain of three runs through tpuhip_conv2d_chain3_i8");
  const bool add = f && f->enable;
  if (ch->kind == 2) {
    TPUHIP_REQUIRE(!add, "conv chain: a depthwise -> pointwise chain takes its add behind the second conv "
                         "(tpuhip_conv2d_chain_post_i8)");
    return dwpw_run(ctx, ch, x, y_a, nullptr, y_b, nullptr);
  }
  TPUHIP_REQUIRE(!add || add_src, "conv chain: fused add without its other operand");
  if (add) {
    TPUHIP_REQUIRE(f->rshift >= 0 && f->rshift <= 30, "conv chain: add rshift %d outside [0,30]", f->rshift);
    TPUHIP_REQUIRE(f->m_src >= -128 && f->m_src <= 127 && f->m_conv >= -128 && f->m_conv <= 127,
                   "conv chain: add multipliers must be int8");
  }
  const tpuhip_conv_desc &da = ch->da;
  ChainArgs a{};
  a.x = (const int8_t *)x;
  a.w1 = ch->w1;
  a.w2 = ch->w2;
  a.q1 = ch->q1;
  a.q2 = ch->q2;
  a.y_a = (int8_t *)y_a;
  a.add_src = add ? (const int8_t *)add_src : nullptr;
  a.add_dst = add ? (int8_t *)add_out : nullptr;
  a.y_b = (int8_t *)y_b;
  a.npix = da.n * da.oh * da.ow;
  a.x_cs = da.x_cs;
  a.x_bytes = (uint32_t)((int64_t)a.npix * da.x_cs);
  a.lo1 = da.do_relu ? 0 : -128;
  a.lo2 = ch->db.do_relu ? 0 : -128;
#ifdef TPUHIP_TRACE
  a.trace = getenv("TPUHIP_TRACE_PTR") ? (unsigned long long *)strtoull(getenv("TPUHIP_TRACE_PTR"), nullptr, 16) : nullptr;
#endif
  if (add) {
    a.add_m_src = f->m_src;
    a.add_m_conv = f->m_conv;
    a.add_rshift = f->rshift;
    a.add_relu = f->do_relu ? 1 : 0;
    a.add_pk = std::abs(f->m_src) <= 127 && std::abs(f->m_conv) <= 127 && f->rshift <= 8;
  }
  switch (ch->variant) {
#define X(i, OC1, KP1, OC2, BN, O, L)                                                                      \
  case i: {                                                                                                \
    auto kernel = conv_chain_kernel<OC1, KP1, OC2, BN, O, L>;                                              \
    constexpr unsigned lds = chain_lds_bytes<OC1, KP1, OC2, BN, L>();                                      \
    TPUHIP_REQUIRE(raise_dynamic_lds((const void *)kernel, lds), "conv chain: raising the LDS limit failed"); \
    const int per_cu = std::max(1, std::min((int)(160u * 1024 / lds), O / 2));                             \
    const int slots = ctx->num_cu * per_cu;                                                                \
    /* whole rounds of BN-pixel tiles over the resident workgroups; what is left runs as 32-pixel */       \
    /* tiles if one round of those covers it (half a round's time instead of a whole one), else as */      \
    /* BN-pixel tiles with the ragged end in 32-pixel tiles */                                             \
    a.n_full = a.npix / BN / slots * slots;                                                                \
    if (BN == 32 || a.npix - a.n_full * BN > slots * 32) a.n_full = a.npix / BN;                           \
    a.n_tiles = a.n_full + (a.npix - a.n_full * BN + 31) / 32;                                             \
    const int gsz = std::min(a.n_tiles, slots);                                                            \
    const dim3 grid((unsigned)gsz), block(512);                                                            \
    if (ctx->prof_start)                                                                                   \
      hipExtLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, ctx->prof_start, ctx->prof_stop, 0, a); \
    else                                                                                                   \
      hipLaunchKernelGGL(kernel, grid, block, lds, ctx->stream, a);                                        \
  } break;
    TPUHIP_CHAIN_VARIANTS(X)
#undef X
    default: return set_error(TPUHIP_ERR_INVALID, "conv chain: unknown variant %d", ch->variant);
  }
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // extern "C"

// Host-side pieces shared by the launches that run two convolutions as one (conv_chain.hip: two
// pointwise convs; conv_dwpw.hip: a depthwise conv and the pointwise conv behind it): the handle
// the C ABI hands out, the proof and layout of the overflow-free requantisation planes, and the
// MFMA A-operand fragment order of a [oc][k] filter.
#pragma once

#include "common.hpp"
#include "conv_epilogue.hpp"

#include <cstdlib>
#include <map>
#include <mutex>
#include <string>
#include <vector>

struct tpuhip_conv_chain {
  tpuhip_conv_desc da, db, dc;   // dc: the third conv of an inverted-residual chain
  int kind = 0;      // 1: pointwise -> pointwise, 2: depthwise -> pointwise, 3: pointwise -> depthwise -> pointwise
  int variant = -1;  // index into the kernel variants of the kind
  int kp1 = 0;
  int8_t *w1 = nullptr, *w2 = nullptr, *w3 = nullptr;
  uint32_t *w2d = nullptr;       // kind 3: the depthwise filter as one dword per lane and tap
  int32_t *q1 = nullptr, *q2 = nullptr, *q3 = nullptr;
  std::string name;
};

namespace tpuhip {

inline bool is_pointwise_conv(const tpuhip_conv_desc &d) {
  return d.g == 1 && d.kh == 1 && d.kw == 1 && d.sh == 1 && d.sw == 1 && d.dh == 1 && d.dw == 1 && d.pt == 0 &&
         d.pb == 0 && d.pl == 0 && d.pr == 0 && !d.ins_h && !d.ins_w && !d.relu_first && d.ih == d.oh && d.iw == d.ow;
}

// Per-channel requantisation data of `oc` channels whose filters hold `per_oc` weights each, as the
// five planes the kernels read: (low, high) of the 64-bit addend bias * mult + 2^30 | multiplier |
// shift | 2^(r-1); with a ReLU the short form (addend + 2^(r-1) * 2^31, shift r - 1).  Planes are
// `ocp` >= oc channels long, the rest zero (a zero accumulator then requantises to zero).
// false: the overflow-free form cannot be proved for some channel (a right shift of 0, or sums that
// could overflow the rounding).
inline bool requant_planes(int oc, int ocp, size_t per_oc, bool relu, const int8_t *filter, const int32_t *bias,
                           const int32_t *mult, const int32_t *rshift, std::vector<int32_t> *out) {
  out->assign((size_t)5 * ocp, 0);
  for (int i = 0; i < oc; ++i) {
    if (rshift[i] < 1 || rshift[i] > 31) return false;
    const int32_t b = bias ? bias[i] : 0;
    const int64_t hpot = 1ll << (rshift[i] - 1);
    int64_t sumw = 0;
    for (size_t k = 0; k < per_oc; ++k) sumw += std::abs((int)filter[(size_t)i * per_oc + k]);
    if (128 * sumw + std::llabs((long long)b) + 1 + hpot >= (1ll << 31)) return false;
    int64_t c = (int64_t)b * (int64_t)mult[i] + (1ll << 30);
    if (relu) c += hpot << 31;
    (*out)[2 * i] = (int32_t)(uint32_t)(c & 0xffffffffll);
    (*out)[2 * i + 1] = (int32_t)(c >> 32);
    (*out)[2 * ocp + i] = mult[i];
    (*out)[3 * ocp + i] = rshift[i] - (relu ? 1 : 0);
    (*out)[4 * ocp + i] = (int32_t)hpot;
  }
  return true;
}

// MFMA A-operand fragments of a [oc][ic] filter: [32-channel block][K slice][lane][16 bytes], lane l
// holding MFMA row l & 31 -- channel mfma_row_to_oc(row, tm) of its group of tm blocks -- and K
// bytes 32 * slice + 16 * (l >> 5) .. + 15.  nblk blocks (channels past oc are zero rows), K padded to kp.
inline std::vector<int8_t> mfma_a_fragments(const int8_t *filter, int oc, int nblk, int ic, int kp, int tm) {
  const int ks_n = kp / 32;
  std::vector<int8_t> out((size_t)nblk * ks_n * 1024, 0);
  for (int blk = 0; blk < nblk; ++blk)
    for (int ks = 0; ks < ks_n; ++ks)
      for (int l = 0; l < 64; ++l) {
        const int group0 = blk / tm * tm * 32;
        const int ch = group0 + mfma_row_to_oc((blk % tm) * 32 + (l & 31), tm);
        if (ch >= oc) continue;
        for (int b = 0; b < 16; ++b) {
          const int k = ks * 32 + (l >> 5) * 16 + b;
          if (k < ic) out[((size_t)(blk * ks_n + ks) * 64 + l) * 16 + b] = filter[(size_t)ch * ic + k];
        }
      }
  return out;
}

// raises a kernel's dynamic LDS limit once per kernel and size
inline bool raise_dynamic_lds(const void *kernel, unsigned bytes) {
  static std::mutex mu;
  static std::map<const void *, unsigned> raised;
  std::lock_guard<std::mutex> lock(mu);
  auto it = raised.find(kernel);
  if (it != raised.end() && it->second >= bytes) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes) != hipSuccess) return false;
  raised[kernel] = bytes;
  return true;
}

template <typename T>
inline int upload_vec(tpuhip_ctx *ctx, const std::vector<T> &v, T **dptr) {
  if (int rc = tpuhip_malloc(ctx, v.size() * sizeof(T), (void **)dptr)) return rc;
  return tpuhip_upload(ctx, *dptr, v.data(), v.size() * sizeof(T));
}

// depthwise -> pointwise (conv_dwpw.hip)
bool dwpw_covers(const tpuhip_conv_desc &a, const tpuhip_conv_desc &b);
const char *dwpw_variant_name(int i);   // null past the last one
int dwpw_prepack(tpuhip_ctx *ctx, tpuhip_conv_chain *ch, const int8_t *filter_a, const int32_t *bias_a,
                 const int32_t *mult_a, const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                 const int32_t *mult_b, const int32_t *rshift_b);
int dwpw_run(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y_a, const tpuhip_conv_post *post_a,
             void *y_b, const tpuhip_conv_post *post_b);

// pointwise -> depthwise -> pointwise (conv_irb.hip)
bool irb_covers(const tpuhip_conv_desc &e, const tpuhip_conv_desc &d, const tpuhip_conv_desc &p);
const char *irb_variant_name(int i);    // null past the last one
int irb_prepack(tpuhip_ctx *ctx, tpuhip_conv_chain *ch, const tpuhip_chain_conv *ce, const tpuhip_chain_conv *cd,
                const tpuhip_chain_conv *cp);
int irb_run(tpuhip_ctx *ctx, const tpuhip_conv_chain *ch, const void *x, void *y, const tpuhip_conv_post *post);

}  // namespace tpuhip

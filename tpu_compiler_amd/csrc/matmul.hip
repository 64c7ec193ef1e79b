// Batched and transposed FullyConnected (core/fullyconnected.cpp:44-91; shapes by
// parseFullyConnectedParam, TPUOperationSupport.cpp:568-605) on channels-last device tensors.
// The reference permutes the input into [batch][m][k], runs one inner product per batch and
// permutes the result back; here a lane owns one element of the RESULT in its logical order,
// finds the operands through the tensors' 4-d views, and so needs no permuted copies.  This is
// the general form (any batch, either transpose, results of rank 3 or 4); the plain [m,k] x
// [n,k] case runs on the MFMA path (tpuhip_fc_prepack).
#include "common.hpp"

#include <vector>

using namespace tpuhip;

struct tpuhip_fc_batched_weights {
  tpuhip_fc_batched_desc d;
  int8_t *filter = nullptr;   // [batch][n][k]
  int32_t *params = nullptr;  // bias [batch][n] (zeros without one), then multiplier[batch], rshift[batch]
  int64_t total = 0;          // result elements
};

namespace {

struct FcbArgs {
  tpuhip_fc_batched_desc d;
  const int8_t *x, *w;
  const int32_t *bias, *mult, *rshift;
  int8_t *y;
  int64_t total;
};

// logical flat index of a 4-d view -> byte offset in the channels-last tensor
__device__ __forceinline__ int64_t view_offset(int64_t g, int C, int H, int W, int cs) {
  const int w = (int)(g % W);
  g /= W;
  const int h = (int)(g % H);
  g /= H;
  const int c = (int)(g % C);
  const int64_t n = g / C;
  return ((n * H + h) * W + w) * cs + c;
}

__global__ __launch_bounds__(256) void fc_batched_kernel(FcbArgs a) {
  const tpuhip_fc_batched_desc &d = a.d;
  const int64_t mn = (int64_t)d.m * d.n;
  for (int64_t f = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; f < a.total;
       f += (int64_t)gridDim.x * blockDim.x) {
    // the result's logical index: [batch_high][m][batch_low][n] when transposed, else [batch][m][n]
    int64_t r = f;
    const int nn = (int)(r % d.n);
    r /= d.n;
    int hb, lb, mm;
    if (d.output_transpose) {
      lb = (int)(r % d.batch_low);
      r /= d.batch_low;
      mm = (int)(r % d.m);
      hb = (int)(r / d.m);
    } else {
      mm = (int)(r % d.m);
      r /= d.m;
      lb = (int)(r % d.batch_low);
      hb = (int)(r / d.batch_low);
    }
    const int b = hb * d.batch_low + lb;
    // first element of the input row: [batch_high][m][batch_low][k] when transposed, else [batch][m][k]
    const int64_t g0 = d.input_transpose ? (((int64_t)hb * d.m + mm) * d.batch_low + lb) * d.k
                                         : ((int64_t)b * d.m + mm) * d.k;
    const int64_t x0 = view_offset(g0, d.x_c, d.x_h, d.x_w, d.x_cs);
    const int64_t xs = d.k > 1 ? view_offset(g0 + 1, d.x_c, d.x_h, d.x_w, d.x_cs) - x0 : 0;
    const int8_t *wr = a.w + ((int64_t)b * d.n + nn) * d.k;
    const int8_t *xr = a.x + x0;
    int32_t s = a.bias[(int64_t)b * d.n + nn];
    for (int t = 0; t < d.k; ++t) s += (int32_t)xr[(int64_t)t * xs] * (int32_t)wr[t];
    if (d.do_relu) s = max(s, 0);
    // (rshift, multiplier) of block f / (m*n) of the result as it lies after the output permute (:78-87)
    const int i = (int)(f / mn);
    const int32_t e = a.rshift[i];
    const int32_t mask = (int32_t)((1u << e) - 1u);
    a.y[view_offset(f, d.y_c, d.y_h, d.y_w, d.y_cs)] =
        (int8_t)requant_qdm(s, a.mult[i], e, mask, mask >> 1, -128);
  }
}

bool last_dim_is(int c, int h, int w, int want) {
  if (want == 1) return true;
  const int last = w > 1 ? w : h > 1 ? h : c;
  return last == want;
}

}  // namespace

extern "C" {

int tpuhip_fc_batched_prepack(tpuhip_ctx *ctx, const tpuhip_fc_batched_desc *desc, const int8_t *filter,
                              const int32_t *bias, const int32_t *multiplier, const int32_t *rshift,
                              tpuhip_fc_batched_weights **out) {
  TPUHIP_REQUIRE(ctx && desc && filter && multiplier && rshift && out, "tpuhip_fc_batched_prepack: NULL argument");
  const tpuhip_fc_batched_desc &d = *desc;
  TPUHIP_REQUIRE(d.batch_high >= 1 && d.batch_low >= 1 && d.m >= 1 && d.k >= 1 && d.n >= 1,
                 "fc_batched: batch_high, batch_low, m, k, n must be positive");
  const int64_t batch = (int64_t)d.batch_high * d.batch_low;
  TPUHIP_REQUIRE(batch * d.m * (int64_t)d.k < (1ll << 31) && batch * d.m * (int64_t)d.n < (1ll << 31) &&
                     batch * d.n * (int64_t)d.k < (1ll << 31),
                 "fc_batched: tensor of 2^31 elements or more");
  TPUHIP_REQUIRE(d.x_c >= 1 && d.x_h >= 1 && d.x_w >= 1 && d.y_c >= 1 && d.y_h >= 1 && d.y_w >= 1,
                 "fc_batched: 4-d views must be positive");
  TPUHIP_REQUIRE(d.x_cs >= d.x_c && d.y_cs >= d.y_c, "fc_batched: channel stride below the channel count");
  TPUHIP_REQUIRE((batch * d.m * d.k) % ((int64_t)d.x_c * d.x_h * d.x_w) == 0,
                 "fc_batched: the input's view (%d,%d,%d) does not divide batch*m*k", d.x_c, d.x_h, d.x_w);
  TPUHIP_REQUIRE((batch * d.m * d.n) % ((int64_t)d.y_c * d.y_h * d.y_w) == 0,
                 "fc_batched: the result's view (%d,%d,%d) does not divide batch*m*n", d.y_c, d.y_h, d.y_w);
  TPUHIP_REQUIRE(last_dim_is(d.x_c, d.x_h, d.x_w, d.k), "fc_batched: the input's last dim must be k = %d", d.k);
  TPUHIP_REQUIRE(last_dim_is(d.y_c, d.y_h, d.y_w, d.n), "fc_batched: the result's last dim must be n = %d", d.n);
  for (int64_t i = 0; i < batch; ++i)
    TPUHIP_REQUIRE(rshift[i] >= 0 && rshift[i] <= 31, "fc_batched: rshift[%lld] = %d outside [0,31]",
                   (long long)i, rshift[i]);
  TPUHIP_CHECK_HIP(hipSetDevice(ctx->device));
  auto *w = new tpuhip_fc_batched_weights;
  w->d = d;
  w->total = batch * d.m * d.n;
  const size_t fbytes = (size_t)(batch * d.n * d.k);
  std::vector<int32_t> params((size_t)(batch * d.n + 2 * batch), 0);
  if (bias) std::copy(bias, bias + batch * d.n, params.begin());
  std::copy(multiplier, multiplier + batch, params.begin() + batch * d.n);
  std::copy(rshift, rshift + batch, params.begin() + batch * d.n + batch);
  hipError_t e = hipMalloc((void **)&w->filter, fbytes);
  if (e == hipSuccess) e = hipMalloc((void **)&w->params, params.size() * sizeof(int32_t));
  if (e == hipSuccess) e = hipMemcpy(w->filter, filter, fbytes, hipMemcpyHostToDevice);
  if (e == hipSuccess)
    e = hipMemcpy(w->params, params.data(), params.size() * sizeof(int32_t), hipMemcpyHostToDevice);
  if (e != hipSuccess) {
    tpuhip_fc_batched_destroy(ctx, w);
    return set_error(TPUHIP_ERR_HIP, "fc_batched: uploading the weights failed: %s", hipGetErrorString(e));
  }
  *out = w;
  return TPUHIP_OK;
}

int tpuhip_fc_batched_destroy(tpuhip_ctx *ctx, tpuhip_fc_batched_weights *w) {
  (void)ctx;
  if (!w) return TPUHIP_OK;
  if (w->filter) (void)hipFree(w->filter);
  if (w->params) (void)hipFree(w->params);
  delete w;
  return TPUHIP_OK;
}

int tpuhip_fc_batched_i8(tpuhip_ctx *ctx, const tpuhip_fc_batched_weights *w, const void *x, void *y) {
  TPUHIP_REQUIRE(ctx && w && x && y, "tpuhip_fc_batched_i8: NULL argument");
  const int64_t batch = (int64_t)w->d.batch_high * w->d.batch_low;
  FcbArgs a;
  a.d = w->d;
  a.x = static_cast<const int8_t *>(x);
  a.w = w->filter;
  a.bias = w->params;
  a.mult = w->params + batch * w->d.n;
  a.rshift = a.mult + batch;
  a.y = static_cast<int8_t *>(y);
  a.total = w->total;
  const unsigned blocks = (unsigned)std::min<int64_t>(ceil_div64(a.total, 256), (int64_t)ctx->num_cu * 32);
  launch(ctx, fc_batched_kernel, dim3(blocks), dim3(256), a);
  TPUHIP_CHECK_HIP(hipGetLastError());
  return TPUHIP_OK;
}

}  // extern "C"

/*
 * TEST INFRASTRUCTURE ONLY -- see tpu_oracle.h.  CPU restatement of the
 * tpuc-interpreter INT8 arithmetic; the checker for the HIP kernels.
 *
 * Build: make -C oracle   (gcc, -ffp-contract=off so no fused multiply-add
 * can change a float result).
 */
#include "tpu_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

/* ------------------------------------------------------------------------- */
/* scalar arithmetic                                                          */
/* ------------------------------------------------------------------------- */

/* QuantizationArithmetic.cpp:501-509.  C '/' truncates toward zero; with the
 * sign-dependent nudge this rounds a*b/2^31 to nearest, ties toward +inf.  The
 * final static_cast keeps the low 32 bits. */
int32_t orc_srdhm(int32_t a, int32_t b) {
  int64_t ab = (int64_t)a * (int64_t)b;
  int32_t nudge = ab >= 0 ? (1 << 30) : (1 - (1 << 30));
  int64_t q = (ab + nudge) / (1ll << 31);
  return (int32_t)(uint32_t)(uint64_t)q;
}

/* QuantizationArithmetic.cpp:487-499 */
int32_t orc_rdbp(int32_t x, int exponent) {
  if (x == 0) return 0;
  if (exponent == 0) return x;
  if (exponent < 0 || exponent > 31) return x; /* outside the reference's assert */
  const int32_t mask = (int32_t)((1ll << exponent) - 1);
  const int32_t remainder = x & mask;
  const int32_t threshold = (mask >> 1) + ((x < 0) ? 1 : 0);
  return (x >> exponent) + ((remainder > threshold) ? 1 : 0);
}

/* QuantizationArithmetic.cpp:301-334: "int q = floor(f + 0.5)" -- the sum is
 * formed in double (0.5 is a double literal), so it is exact. */
int8_t orc_saturate_int8(float f) {
  double s = floor((double)f + 0.5);
  int q;
  /* the reference converts the double to int; outside int range that is
   * undefined, x86 yields INT_MIN.  Clamp first: same result wherever the
   * reference's is defined, and saturation for the rest. */
  if (s > 127.0)
    q = 127;
  else if (s < -128.0)
    q = -128;
  else
    q = (int)s;
  return (int8_t)q;
}

/* QuantizationArithmetic.cpp:481-483: v / (1 << rshift) in float */
int8_t orc_apply_rshift_sat8(float v, uint32_t rshift) {
  return orc_saturate_int8(v / (float)(1 << rshift));
}

/* QuantizationArithmetic.cpp:518-528 */
int8_t orc_apply_mult_rshift_sat8_f(float v, uint32_t rshift, uint32_t multiplier, int qdm) {
  if (qdm) {
    int32_t q = orc_rdbp(orc_srdhm((int32_t)v, (int32_t)multiplier), (int)rshift);
    return orc_saturate_int8((float)q);
  }
  /* float * uint32 -> float product, then float / int -> float quotient */
  float prod = v * (float)multiplier;
  return orc_saturate_int8(prod / (float)(1 << rshift));
}

/* QuantizationArithmetic.cpp:530-539.  Without qdm "v * multiplier" is int32 *
 * uint32, i.e. unsigned arithmetic, and so is the division. */
int8_t orc_apply_mult_rshift_sat8_i(int32_t v, uint32_t rshift, uint32_t multiplier, int qdm) {
  if (qdm) {
    int32_t q = orc_rdbp(orc_srdhm(v, (int32_t)multiplier), (int)rshift);
    return orc_saturate_int8((float)q);
  }
  uint32_t prod = (uint32_t)v * multiplier;
  uint32_t quo = prod / (uint32_t)(1 << rshift);
  return orc_saturate_int8((float)quo);
}

uint32_t orc_f2u32(float f) { return (uint32_t)(uint64_t)(int64_t)f; }

/* ------------------------------------------------------------------------- */
/* convolution                                                                */
/* ------------------------------------------------------------------------- */

/* The reference pads with zeros (MKL-DNN convolution, conv.cpp ignores
 * pad_value) and inserts ins_h / ins_w zeros between input samples
 * (my_dilateActivation, NativeCpuImplementation.cpp:480-503).  Both are done
 * here by materialising the dilated, padded planes once; the contraction then
 * runs over plain in-bounds windows.  For stride 1 a tap contributes to the
 * whole output plane (kept at the padded row pitch) as one long vector
 * operation, which is what makes full-size graphs checkable in seconds. */
#define CONV_BODY(ACC_T, X_T, W_T, MUL)                                                     \
  const int icg = d->ic / d->g, ocg = d->oc / d->g;                                         \
  const int ihd = (d->ih - 1) * (d->ins_h + 1) + 1;                                         \
  const int iwd = (d->iw - 1) * (d->ins_w + 1) + 1;                                         \
  const int ihp = ihd + d->pt + d->pb, iwp = iwd + d->pl + d->pr;                           \
  const int64_t plane = (int64_t)ihp * iwp;                                                 \
  /* rows the windows may touch beyond ihp when oh was rounded up by the importer */       \
  const int need_h = (d->oh - 1) * d->sh + (d->kh - 1) * d->dh + 1;                         \
  const int need_w = (d->ow - 1) * d->sw + (d->kw - 1) * d->dw + 1;                         \
  if (need_h > ihp || need_w > iwp) abort(); /* caller passed an impossible output size */ \
  X_T *xp = (X_T *)calloc((size_t)d->n * d->ic * plane + 64, sizeof(X_T));                  \
  _Pragma("omp parallel for")                                                               \
  for (int64_t nc = 0; nc < (int64_t)d->n * d->ic; ++nc)                                    \
    for (int h = 0; h < d->ih; ++h)                                                         \
      for (int w_ = 0; w_ < d->iw; ++w_)                                                    \
        xp[nc * plane + (int64_t)(d->pt + h * (d->ins_h + 1)) * iwp + d->pl +               \
           w_ * (d->ins_w + 1)] = x[(nc * d->ih + h) * d->iw + w_];                         \
  const int64_t osz = (int64_t)d->oh * d->ow;                                               \
  const int64_t span = (int64_t)(d->oh - 1) * iwp + d->ow; /* stride-1 plane at pitch iwp */ \
  _Pragma("omp parallel")                                                                   \
  {                                                                                         \
    ACC_T *ap = (ACC_T *)malloc(sizeof(ACC_T) * (size_t)(d->oh * (int64_t)iwp + 64));       \
    _Pragma("omp for collapse(2) schedule(dynamic, 1)")                                     \
    for (int n = 0; n < d->n; ++n) {                                                        \
      for (int oc = 0; oc < d->oc; ++oc) {                                                  \
        const int gi = oc / ocg;                                                            \
        const int unit = (d->sh == 1 && d->sw == 1);                                        \
        if (unit) {                                                                         \
          for (int64_t i = 0; i < span; ++i) ap[i] = 0;                                     \
        } else {                                                                            \
          for (int64_t i = 0; i < osz; ++i) ap[i] = 0;                                      \
        }                                                                                   \
        for (int c = 0; c < icg; ++c) {                                                     \
          const X_T *xc = xp + ((int64_t)n * d->ic + (int64_t)gi * icg + c) * plane;        \
          for (int kh = 0; kh < d->kh; ++kh) {                                              \
            for (int kw = 0; kw < d->kw; ++kw) {                                            \
              const W_T wv = w[(((int64_t)oc * icg + c) * d->kh + kh) * d->kw + kw];        \
              if (wv == 0) continue;                                                        \
              const X_T *xt = xc + (int64_t)kh * d->dh * iwp + kw * d->dw;                  \
              if (unit) {                                                                   \
                for (int64_t i = 0; i < span; ++i) ap[i] += MUL(wv, xt[i]);                 \
              } else {                                                                      \
                for (int oh = 0; oh < d->oh; ++oh) {                                        \
                  const X_T *xr = xt + (int64_t)oh * d->sh * iwp;                           \
                  ACC_T *ar = ap + (int64_t)oh * d->ow;                                     \
                  for (int ow = 0; ow < d->ow; ++ow) ar[ow] += MUL(wv, xr[ow * d->sw]);     \
                }                                                                           \
              }                                                                             \
            }                                                                               \
          }                                                                                 \
        }                                                                                   \
        ACC_T *a = acc + ((int64_t)n * d->oc + oc) * osz;                                   \
        if (unit) {                                                                         \
          for (int oh = 0; oh < d->oh; ++oh)                                                \
            for (int ow = 0; ow < d->ow; ++ow) a[oh * d->ow + ow] = ap[(int64_t)oh * iwp + ow]; \
        } else {                                                                            \
          for (int64_t i = 0; i < osz; ++i) a[i] = ap[i];                                   \
        }                                                                                   \
      }                                                                                     \
    }                                                                                       \
    free(ap);                                                                               \
  }                                                                                         \
  free(xp);

#define MUL_I32(a, b) ((int32_t)(a) * (int32_t)(b))
#define MUL_ABS(a, b) (abs((int32_t)(a)) * abs((int32_t)(b)))
#define MUL_F32(a, b) ((a) * (b))

/* include/tpuc/NativeCpuImplementation.h:11-102 (MKL-DNN convolution_direct,
 * zero padding, dilation passed as d-1, groups) restated as the integer
 * cross-correlation it computes inside the exact domain. */
void orc_conv2d_acc(const int8_t *x, const int8_t *w, int32_t *acc, const orc_conv_desc *d) {
  CONV_BODY(int32_t, int8_t, int8_t, MUL_I32)
}

static void conv2d_abs(const int8_t *x, const int8_t *w, int32_t *acc, const orc_conv_desc *d) {
  CONV_BODY(int32_t, int8_t, int8_t, MUL_ABS)
}

void orc_conv2d_acc_f32(const float *x, const float *w, float *acc, const orc_conv_desc *d) {
  CONV_BODY(float, float, float, MUL_F32)
}

int64_t orc_conv2d_guard(const int8_t *x, const int8_t *w, const orc_conv_desc *d) {
  const int64_t total = (int64_t)d->n * d->oc * d->oh * d->ow;
  int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)total);
  conv2d_abs(x, w, acc, d);
  int64_t m = 0;
  for (int64_t i = 0; i < total; ++i)
    if (acc[i] > m) m = acc[i];
  free(acc);
  return m;
}

/* QuantizationArithmetic.cpp:849-871 */
void orc_requant_per_channel(const int32_t *acc, int8_t *y, const float *bias, int do_relu,
                             int64_t on, int64_t oc, int64_t isz, const float *rshift,
                             const float *multiplier) {
#pragma omp parallel for collapse(2)
  for (int64_t n = 0; n < on; ++n) {
    for (int64_t i = 0; i < oc; ++i) {
      /* the float -> uint32_t conversions happen at the call (:863-865) */
      const uint32_t rs = orc_f2u32(rshift[i]);
      const uint32_t mu = orc_f2u32(multiplier[i]);
      const int32_t b = bias ? (int32_t)bias[i] : 0;
      for (int64_t j = 0; j < isz; ++j) {
        int32_t v = acc[n * oc * isz + i * isz + j];
        v = (int32_t)((uint32_t)v + (uint32_t)b);
        v = orc_apply_mult_rshift_sat8_i(v, rs, mu, 1);
        if (do_relu && v < 0) v = 0;
        y[n * oc * isz + i * isz + j] = (int8_t)v;
      }
    }
  }
}

/* conv.cpp:80-104, INT8 branch.  The MKL-DNN conv runs with a zero bias
 * (:57-65); the int32 bias is added in the epilogue.  Without with_bias the
 * epilogue adds a zero tensor (:59-61). */
void orc_conv2d_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                   const float *multiplier, int8_t *y, const orc_conv_desc *d) {
  const int64_t total = (int64_t)d->n * d->oc * d->oh * d->ow;
  int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * (size_t)total);
  orc_conv2d_acc(x, w, acc, d);
  orc_requant_per_channel(acc, y, d->with_bias ? bias : NULL, d->do_relu, d->n, d->oc,
                          (int64_t)d->oh * d->ow, rshift, multiplier);
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* fully connected                                                            */
/* ------------------------------------------------------------------------- */

/* fullyconnected.cpp:44-91: inner product (weights n x k, NativeCpuImplementation.cpp:185-288)
 * with the bias added inside the fp32 primitive, ReLU on the float sums, then
 * one qdm requant per batch matmul (rshift_data->at(i), multiplier_data->at(i)).
 * Inside the exact domain the fp32 sum equals the integer sum, which is what
 * is computed here. */
void orc_fc_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
               const float *multiplier, int8_t *y, int batch, int m, int k, int n, int do_relu) {
  for (int b = 0; b < batch; ++b) {
    const uint32_t rs = orc_f2u32(rshift[b]);
    const uint32_t mu = orc_f2u32(multiplier[b]);
#pragma omp parallel for collapse(2)
    for (int i = 0; i < m; ++i) {
      for (int j = 0; j < n; ++j) {
        const int8_t *xr = x + ((int64_t)b * m + i) * k;
        const int8_t *wr = w + ((int64_t)b * n + j) * k;
        int32_t s = 0;
        for (int t = 0; t < k; ++t) s += (int32_t)xr[t] * (int32_t)wr[t];
        float f = (float)s;
        if (bias) f = (float)(s + (int32_t)bias[(int64_t)b * n + j]);
        if (do_relu && !(f > 0)) f = 0;
        y[((int64_t)b * m + i) * n + j] = orc_apply_mult_rshift_sat8_f(f, rs, mu, 1);
      }
    }
  }
}

/* fullyconnected.cpp:44-91 with the batch loop and both transposes: x in the input's logical
 * order ([batch_high][m][batch_low][k] under input_transpose, my_permute(0,2,1,3) at :53-57, else
 * [batch][m][k]); one inner product per batch b = hb*batch_low + lb with filter block b and bias
 * block b (:62-68); under output_transpose the [batch_high][batch_low][m][n] sums are permuted to
 * [batch_high][m][batch_low][n] (:69-72); ReLU (:73-75); then element f of the RESULT AS IT LIES
 * takes rshift / multiplier number f / (m*n) (:77-88) -- after an output permute that is not the
 * matmul's own batch index. */
void orc_fc_batched_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                       const float *multiplier, int8_t *y, int batch_high, int batch_low, int m,
                       int k, int n, int ltrans, int otrans, int do_relu) {
  const int batch = batch_high * batch_low;
  const int64_t isz = (int64_t)m * n;
  float *sum = (float *)malloc(sizeof(float) * (size_t)(batch * isz));
#pragma omp parallel for collapse(2)
  for (int b = 0; b < batch; ++b)
    for (int i = 0; i < m; ++i) {
      const int hb = b / batch_low, lb = b % batch_low;
      const int8_t *xr = ltrans ? x + ((((int64_t)hb * m + i) * batch_low + lb) * k)
                                : x + ((int64_t)b * m + i) * k;
      for (int j = 0; j < n; ++j) {
        const int8_t *wr = w + ((int64_t)b * n + j) * k;
        int32_t s = 0;
        for (int t = 0; t < k; ++t) s += (int32_t)xr[t] * (int32_t)wr[t];
        if (bias) s += (int32_t)bias[(int64_t)b * n + j];
        const int64_t at = otrans ? ((((int64_t)hb * m + i) * batch_low + lb) * n + j)
                                  : (((int64_t)b * m + i) * n + j);
        sum[at] = (float)s;
      }
    }
  for (int64_t f = 0; f < batch * isz; ++f) {
    float v = sum[f];
    if (do_relu && !(v > 0)) v = 0;
    const int i = (int)(f / isz);
    y[f] = orc_apply_mult_rshift_sat8_f(v, orc_f2u32(rshift[i]), orc_f2u32(multiplier[i]), 1);
  }
  free(sum);
}

int64_t orc_fc_guard(const int8_t *x, const int8_t *w, const float *bias, int batch, int m, int k,
                     int n) {
  int64_t worst = 0;
  for (int b = 0; b < batch; ++b)
    for (int i = 0; i < m; ++i)
      for (int j = 0; j < n; ++j) {
        const int8_t *xr = x + ((int64_t)b * m + i) * k;
        const int8_t *wr = w + ((int64_t)b * n + j) * k;
        int64_t s = 0;
        for (int t = 0; t < k; ++t) s += llabs((int64_t)xr[t] * wr[t]);
        if (bias) s += llabs((int64_t)bias[(int64_t)b * n + j]);
        if (s > worst) worst = s;
      }
  return worst;
}

/* ------------------------------------------------------------------------- */
/* eltwise add                                                                */
/* ------------------------------------------------------------------------- */

/* eltwise.cpp:52-85: each input times (int8_t)multiplier[i] in float, summed
 * in float, ReLU, then v / 2^rshift[0] in float and floor(.+0.5), saturate. */
void orc_eltwise_add_i8(const int8_t *const *xs, int nin, const float *multiplier,
                        const float *rshift, int do_relu, int8_t *y, size_t count) {
  const uint32_t rs = orc_f2u32(rshift[0]);
#pragma omp parallel for
  for (size_t i = 0; i < count; ++i) {
    float s = 0;
    for (int k = 0; k < nin; ++k) {
      float t = (float)xs[k][i];
      t *= (int8_t)(int)multiplier[k];
      s += t;
    }
    if (do_relu) s = s > 0 ? s : 0;
    y[i] = orc_apply_rshift_sat8(s, rs);
  }
}

/* broadcast.cpp:60-75 index arithmetic; eltwise.cpp i8_invoke bodies for the
 * same-shape case (every n_i == n etc.). */
int orc_binary_i8(const int8_t *x0, const int8_t *x1, int8_t *y, const orc_binary_desc *d,
                  const float *multiplier, float rshift) {
  const uint32_t rs = orc_f2u32(rshift);
  const uint32_t mq = orc_f2u32(multiplier[0]);
  if (d->op == ORC_BIN_MUL && rs == 0 && mq == 0) return -1;
  const int8_t m0 = d->op == ORC_BIN_MUL ? 0 : (int8_t)(int)multiplier[0];
  const int8_t m1 = d->op == ORC_BIN_MUL ? 0 : (int8_t)(int)multiplier[1];
#pragma omp parallel for collapse(2)
  for (int n = 0; n < d->n; ++n)
    for (int c = 0; c < d->c; ++c)
      for (int h = 0; h < d->h; ++h)
        for (int w = 0; w < d->w; ++w) {
          const int64_t i0 = (((int64_t)(d->n0 == 1 ? 0 : n) * d->c0 + (d->c0 == 1 ? 0 : c)) * d->h0 +
                              (d->h0 == 1 ? 0 : h)) * d->w0 + (d->w0 == 1 ? 0 : w);
          const int64_t i1 = (((int64_t)(d->n1 == 1 ? 0 : n) * d->c1 + (d->c1 == 1 ? 0 : c)) * d->h1 +
                              (d->h1 == 1 ? 0 : h)) * d->w1 + (d->w1 == 1 ? 0 : w);
          const int64_t o = (((int64_t)n * d->c + c) * d->h + h) * d->w + w;
          float a = (float)x0[i0], b = (float)x1[i1], v;
          if (d->op == ORC_BIN_MUL) {
            v = a * b;
            if (d->do_relu) v = v > 0 ? v : 0;
            y[o] = orc_apply_mult_rshift_sat8_f(v, rs, mq, 1);
            continue;
          }
          a *= m0;
          b *= m1;
          switch (d->op) {
            case ORC_BIN_ADD: v = a + b; break;
            case ORC_BIN_SUB: v = a - b; break;
            case ORC_BIN_MAX: v = a > b ? a : b; break;
            default: v = a < b ? a : b; break;
          }
          if (d->do_relu) v = v > 0 ? v : 0;
          y[o] = orc_apply_rshift_sat8(v, rs);
        }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* pooling                                                                    */
/* ------------------------------------------------------------------------- */

/* pooling.cpp:155-157 -> MKLPooling (NativeCpuImplementation.h:104-174):
 * pooling_max ignores padded positions. */
void orc_pool_max_i8(const int8_t *x, int8_t *y, const orc_pool_desc *d) {
#pragma omp parallel for
  for (int64_t nc = 0; nc < (int64_t)d->n * d->c; ++nc) {
    const int8_t *xp = x + nc * d->ih * d->iw;
    int8_t *yp = y + nc * d->oh * d->ow;
    for (int oh = 0; oh < d->oh; ++oh)
      for (int ow = 0; ow < d->ow; ++ow) {
        int best = -128; /* an all-padding window cannot occur for valid shapes */
        for (int kh = 0; kh < d->kh; ++kh) {
          int ih = oh * d->sh - d->pt + kh;
          if (ih < 0 || ih >= d->ih) continue;
          for (int kw = 0; kw < d->kw; ++kw) {
            int iw = ow * d->sw - d->pl + kw;
            if (iw < 0 || iw >= d->iw) continue;
            int v = xp[ih * d->iw + iw];
            if (v > best) best = v;
          }
        }
        yp[oh * d->ow + ow] = (int8_t)best;
      }
  }
}

/* pooling.cpp:72-82,147-154: depthwise fp32 conv with an all-ones filter and
 * zero padding (MKLInt8AvgPooling, NativeCpuImplementation.h:176-192) = window
 * sum that counts padding as zeros; then the non-qdm float overload with the
 * scalar (uint32_t)rshift / (uint32_t)multiplier. */
void orc_pool_avg_i8(const int8_t *x, int8_t *y, const orc_pool_desc *d, float rshift,
                     float multiplier) {
  const uint32_t rs = orc_f2u32(rshift);
  const uint32_t mu = orc_f2u32(multiplier);
#pragma omp parallel for
  for (int64_t nc = 0; nc < (int64_t)d->n * d->c; ++nc) {
    const int8_t *xp = x + nc * d->ih * d->iw;
    int8_t *yp = y + nc * d->oh * d->ow;
    for (int oh = 0; oh < d->oh; ++oh)
      for (int ow = 0; ow < d->ow; ++ow) {
        int32_t s = 0;
        for (int kh = 0; kh < d->kh; ++kh) {
          int ih = oh * d->sh - d->pt + kh;
          if (ih < 0 || ih >= d->ih) continue;
          for (int kw = 0; kw < d->kw; ++kw) {
            int iw = ow * d->sw - d->pl + kw;
            if (iw < 0 || iw >= d->iw) continue;
            s += xp[ih * d->iw + iw];
          }
        }
        yp[oh * d->ow + ow] = orc_apply_mult_rshift_sat8_f((float)s, rs, mu, 0);
      }
  }
}

/* ------------------------------------------------------------------------- */
/* activations                                                                */
/* ------------------------------------------------------------------------- */

/* activation.cpp:126-153.  rshift is cast explicitly to uint32_t; the
 * multiplier float is converted implicitly at the call. */
void orc_leaky_relu_i8(const int8_t *x, int8_t *y, size_t count, float rshift_pos,
                       float multiplier_pos, float rshift_neg, float multiplier_neg) {
  const int do_pos_scale = (multiplier_pos != 0.0);
#pragma omp parallel for
  for (size_t i = 0; i < count; ++i) {
    float v = (float)x[i];
    if (v > 0) {
      if (do_pos_scale)
        y[i] = orc_apply_mult_rshift_sat8_f(v, orc_f2u32(rshift_pos), orc_f2u32(multiplier_pos), 0);
      else
        y[i] = x[i];
    } else {
      y[i] = orc_apply_mult_rshift_sat8_f(v, orc_f2u32(rshift_neg), orc_f2u32(multiplier_neg), 0);
    }
  }
}

/* activation.cpp:185-224.  First pass: x > 0 keeps x, else slope[channel] * x (float).
 * Second pass: x > 0 -> float overload, non-qdm, multiplier converted implicitly from
 * float to uint32; else applyRShiftAndSaturateInt8. */
void orc_prelu_i8(const int8_t *x, int8_t *y, int n, int c, int hw, const float *slope,
                  float rshift_pos, float multiplier_pos, float rshift_neg) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < n; ++b)
    for (int ch = 0; ch < c; ++ch) {
      const size_t base = ((size_t)b * c + ch) * hw;
      for (int i = 0; i < hw; ++i) {
        const float in = (float)x[base + i];
        if (in > 0)
          y[base + i] = orc_apply_mult_rshift_sat8_f(in, orc_f2u32(rshift_pos),
                                                     orc_f2u32(multiplier_pos), 0);
        else
          y[base + i] = orc_apply_rshift_sat8(slope[ch] * in, orc_f2u32(rshift_neg));
      }
    }
}

/* scale_lut.cpp:15-31: table->at((int)(ci * 256 + x)) with x the float-stored input, which
 * the quantizer defines for inputs 0..255 (QuantizeInt8.cpp:623-657): x is a uint8 tensor. */
void orc_scale_lut_u8(const uint8_t *x, int8_t *y, int n, int c, int hw, const float *table) {
#pragma omp parallel for collapse(2)
  for (int b = 0; b < n; ++b)
    for (int ch = 0; ch < c; ++ch) {
      const size_t base = ((size_t)b * c + ch) * hw;
      for (int i = 0; i < hw; ++i) {
        const float in = (float)x[base + i];
        y[base + i] = (int8_t)table[(int)(ch * 256 + in)];
      }
    }
}

/* activation.cpp:47-53: y0_table_op->at((unsigned char)input).  float ->
 * unsigned char of a negative value keeps the low byte on x86-64 gcc, i.e. the
 * index is the two's-complement byte of the int8 input. */
void orc_lut_i8(const int8_t *x, int8_t *y, size_t count, const float *table256) {
#pragma omp parallel for
  for (size_t i = 0; i < count; ++i) {
    unsigned char idx = (unsigned char)(int)(float)x[i];
    y[i] = (int8_t)table256[idx];
  }
}

/* core/internal.cpp:13-18 */
void orc_relu_i8(const int8_t *x, int8_t *y, size_t count) {
#pragma omp parallel for
  for (size_t i = 0; i < count; ++i) y[i] = x[i] > 0 ? x[i] : 0;
}

/* clip.cpp:29-40 */
void orc_clip_i8(const int8_t *x, int8_t *y, size_t count, float min, float max, float rshift,
                 float multiplier) {
  const uint32_t rs = orc_f2u32(rshift);
  const uint32_t mu = orc_f2u32(multiplier);
#pragma omp parallel for
  for (size_t i = 0; i < count; ++i) {
    float v = (float)x[i];
    float c = fmaxf(min, fminf(v, max)); /* std::max(min, std::min(v, max)) */
    y[i] = orc_apply_mult_rshift_sat8_f(c, rs, mu, 0);
  }
}

/* ------------------------------------------------------------------------- */
/* data movement                                                              */
/* ------------------------------------------------------------------------- */

/* upsample.cpp:20-41 */
void orc_upsample_i8(const int8_t *x, int8_t *y, int n, int c, int ih, int iw, int scale_h,
                     int scale_w) {
  const int h = ih * scale_h, w = iw * scale_w;
#pragma omp parallel for
  for (int64_t nc = 0; nc < (int64_t)n * c; ++nc)
    for (int hi = 0; hi < h; ++hi)
      for (int wi = 0; wi < w; ++wi)
        y[(nc * h + hi) * w + wi] = x[(nc * ih + hi / scale_h) * iw + wi / scale_w];
}

/* concat.cpp:34-90 */
void orc_concat_i8(const int8_t *const *xs, int nin, const int64_t *shapes, int ndim, int axis,
                   const float *rshift, const float *multiplier, int do_relu, int8_t *y) {
  int64_t num_concats = 1;
  for (int i = 0; i < axis; ++i) num_concats *= shapes[i];
  int64_t out_axis = 0;
  for (int k = 0; k < nin; ++k) out_axis += shapes[(int64_t)k * ndim + axis];
  int64_t inner = 1;
  for (int i = axis + 1; i < ndim; ++i) inner *= shapes[i];
  const int64_t concat_output_size = out_axis * inner;
  const int need_quant = rshift != NULL && multiplier != NULL;
  int64_t global_offset = 0;
  for (int k = 0; k < nin; ++k) {
    const int64_t concat_input_size = shapes[(int64_t)k * ndim + axis] * inner;
    for (int64_t c = 0; c < num_concats; ++c) {
      const int8_t *src = xs[k] + c * concat_input_size;
      int8_t *dst = y + global_offset + concat_output_size * c;
      for (int64_t i = 0; i < concat_input_size; ++i) {
        int8_t v = src[i];
        if (need_quant && !(multiplier[k] == 1 && rshift[k] == 0))
          v = orc_apply_mult_rshift_sat8_f((float)v, orc_f2u32(rshift[k]),
                                           orc_f2u32(multiplier[k]), 0);
        dst[i] = v;
      }
    }
    global_offset += concat_input_size;
  }
  if (do_relu) {
    const int64_t total = concat_output_size * num_concats;
    for (int64_t i = 0; i < total; ++i)
      if (y[i] < 0) y[i] = 0;
  }
}

/* ------------------------------------------------------------------------- */
/* pure data movement                                                         */
/* ------------------------------------------------------------------------- */

/* pad.cpp: constant mode copies rows of the (possibly cut) input into the result buffer and
 * touches nothing else: const_val is parsed (:119) and passed down (:139) but never read, so
 * the padding keeps the zeros the result tensor was created with (cpukernel.cpp:75-80).
 * Edge mode replicates the border (h and w only, asserted). */
void orc_pad_i8(const int8_t *x, int8_t *y, const int64_t *is, const int *pads, int edge_mode) {
  const int8_t const_val = 0;
  const int in = (int)is[0], ic = (int)is[1], ih = (int)is[2], iw = (int)is[3];
  const int on = pads[0] + pads[4] + in, oc = pads[1] + pads[5] + ic;
  const int oh = pads[2] + pads[6] + ih, ow = pads[3] + pads[7] + iw;
  for (int64_t i = 0; i < (int64_t)on * oc * oh * ow; ++i) y[i] = const_val;
  if (edge_mode) {
    for (int n = 0; n < in; ++n)
      for (int c = 0; c < ic; ++c)
        for (int h = 0; h < oh; ++h)
          for (int w = 0; w < ow; ++w) {
            int sh = h - pads[2], sw = w - pads[3];
            sh = sh < 0 ? 0 : sh >= ih ? ih - 1 : sh;
            sw = sw < 0 ? 0 : sw >= iw ? iw - 1 : sw;
            y[(((int64_t)n * oc + c) * oh + h) * ow + w] = x[(((int64_t)n * ic + c) * ih + sh) * iw + sw];
          }
    return;
  }
  const int s_n = pads[0] < 0 ? -pads[0] : 0, s_c = pads[1] < 0 ? -pads[1] : 0;
  const int s_h = pads[2] < 0 ? -pads[2] : 0, s_w = pads[3] < 0 ? -pads[3] : 0;
  const int e_n = pads[4] < 0 ? in + pads[4] : in, e_c = pads[5] < 0 ? ic + pads[5] : ic;
  const int e_h = pads[6] < 0 ? ih + pads[6] : ih, e_w = pads[7] < 0 ? iw + pads[7] : iw;
  const int b_n = pads[0] < 0 ? 0 : pads[0], b_c = pads[1] < 0 ? 0 : pads[1];
  const int b_h = pads[2] < 0 ? 0 : pads[2], b_w = pads[3] < 0 ? 0 : pads[3];
  for (int n = s_n; n < e_n; ++n)
    for (int c = s_c; c < e_c; ++c)
      for (int h = s_h; h < e_h; ++h)
        for (int w = s_w; w < e_w; ++w)
          y[((((int64_t)(n - s_n + b_n)) * oc + (c - s_c + b_c)) * oh + (h - s_h + b_h)) * ow +
            (w - s_w + b_w)] = x[(((int64_t)n * ic + c) * ih + h) * iw + w];
}

void orc_crop_i8(const int8_t *x, int8_t *y, const int64_t *is, const int64_t *os, const int *off,
                 const int *st) {
  for (int64_t n = 0; n < os[0]; ++n)
    for (int64_t c = 0; c < os[1]; ++c)
      for (int64_t h = 0; h < os[2]; ++h)
        for (int64_t w = 0; w < os[3]; ++w) {
          const int64_t a = n * st[0] + off[0], b = c * st[1] + off[1], d = h * st[2] + off[2],
                        e = w * st[3] + off[3];
          y[((n * os[1] + c) * os[2] + h) * os[3] + w] = x[((a * is[1] + b) * is[2] + d) * is[3] + e];
        }
}

void orc_permute_i8(const int8_t *x, int8_t *y, const int64_t *is, const int *order) {
  for (int64_t n = 0; n < is[0]; ++n)
    for (int64_t c = 0; c < is[1]; ++c)
      for (int64_t h = 0; h < is[2]; ++h)
        for (int64_t w = 0; w < is[3]; ++w) {
          const int64_t cur[4] = {n, c, h, w};
          const int64_t in_idx = w + h * is[3] + c * is[2] * is[3] + n * is[1] * is[2] * is[3];
          const int64_t out_idx = cur[order[3]] + cur[order[2]] * is[order[3]] +
                                  cur[order[1]] * is[order[3]] * is[order[2]] +
                                  cur[order[0]] * is[order[3]] * is[order[2]] * is[order[1]];
          y[out_idx] = x[in_idx];
        }
}

void orc_reorg_i8(const int8_t *x, int8_t *y, const int64_t *is, int stride) {
  const int n = (int)is[0], in_c = (int)is[1], in_h = (int)is[2], in_w = (int)is[3];
  const int out_c = in_c * stride * stride, out_h = in_h / stride, out_w = in_w / stride;
  for (int b = 0; b < n; b++)
    for (int k = 0; k < out_c; k++)
      for (int j = 0; j < out_h; j++)
        for (int i = 0; i < out_w; i++) {
          const int64_t in_index = i + out_w * (j + out_h * (k + (int64_t)out_c * b));
          const int c2 = k % in_c, offset = k / in_c;
          const int w2 = i * stride + offset % stride, h2 = j * stride + offset / stride;
          const int64_t out_index = w2 + in_w * (h2 + in_h * (c2 + (int64_t)in_c * b));
          y[in_index] = x[out_index];
        }
}

void orc_tile_i8(const int8_t *x, int8_t *y, const int64_t *is, int axis, int tiles) {
  int64_t outer = 1, inner = 1;
  for (int i = 0; i < axis; ++i) outer *= is[i];
  for (int i = axis; i < 4; ++i) inner *= is[i];
  for (int64_t o = 0; o < outer; ++o)
    for (int t = 0; t < tiles; ++t)
      memcpy(y + o * tiles * inner + t * inner, x + o * inner, (size_t)inner);
}

void orc_reverse_i8(const int8_t *x, int8_t *y, const int64_t *s, int axis) {
  const int64_t stride[4] = {s[1] * s[2] * s[3], s[2] * s[3], s[3], 1};
  for (int64_t n = 0; n < s[0]; ++n)
    for (int64_t c = 0; c < s[1]; ++c)
      for (int64_t h = 0; h < s[2]; ++h)
        for (int64_t w = 0; w < s[3]; ++w) {
          int64_t src[4] = {n, c, h, w}, dst[4] = {n, c, h, w};
          dst[axis] = s[axis] - src[axis] - 1;
          y[dst[0] * stride[0] + dst[1] * stride[1] + dst[2] * stride[2] + dst[3]] =
              x[src[0] * stride[0] + src[1] * stride[1] + src[2] * stride[2] + src[3]];
        }
}

/* Dilate as DilateOpKernel::invoke runs it (core/dilate.cpp:11-33, 51-59: no pads, nothing
 * inserted after the last row / column): the input lands on every (ins_h+1)-th row and
 * (ins_w+1)-th column of the result, everything else is the fill value. */
void orc_dilate_i8(const int8_t *x, int8_t *y, const int64_t *s, int ins_h, int ins_w, int fill) {
  const int64_t planes = s[0] * s[1], h = s[2], w = s[3];
  const int64_t step_h = ins_h + 1, step_w = ins_w + 1;
  const int64_t oh = (h - 1) * step_h + 1, ow = (w - 1) * step_w + 1;
  for (int64_t p = 0; p < planes; ++p) {
    const int8_t *src = x + p * h * w;
    int8_t *dst = y + p * oh * ow;
    for (int64_t r = 0; r < oh; ++r)
      for (int64_t c = 0; c < ow; ++c) {
        const int on_grid = r % step_h == 0 && c % step_w == 0;
        dst[r * ow + c] = on_grid ? src[(r / step_h) * w + c / step_w] : (int8_t)fill;
      }
  }
}

/* ReflectionPad (core/reflectionpad.cpp:21-46): the last dimension grows by pad_l + pad_r; the
 * new columns mirror the row about its first / last element, which is not repeated. */
void orc_reflection_pad_i8(const int8_t *x, int8_t *y, const int64_t *s, int pad_l, int pad_r) {
  const int64_t rows = s[0] * s[1] * s[2], w = s[3], ow = w + pad_l + pad_r;
  for (int64_t r = 0; r < rows; ++r) {
    const int8_t *src = x + r * w;
    int8_t *dst = y + r * ow;
    memcpy(dst + pad_l, src, (size_t)w);
    for (int64_t d = 1; d <= pad_l; ++d) dst[pad_l - d] = src[d];             /* left: 1, 2, ... outwards */
    for (int64_t d = 1; d <= pad_r; ++d) dst[pad_l + w - 1 + d] = src[w - 1 - d];
  }
}

void orc_shuffle_channel_i8(const int8_t *x, int8_t *y, const int64_t *s, int group) {
  const int64_t frame = s[2] * s[3], batch = frame * s[1];
  const int col = (int)(s[1] / group);
  for (int64_t i = 0; i < s[0]; ++i)
    for (int j = 0; j < group; ++j)
      for (int k = 0; k < col; ++k)
        memcpy(y + i * batch + ((int64_t)k * group + j) * frame,
               x + i * batch + ((int64_t)j * col + k) * frame, (size_t)frame);
}

void orc_depth_to_space_i8(const int8_t *x, int8_t *y, const int64_t *is, int r, int dcr_mode) {
  const int in = (int)is[0], ic = (int)is[1], ih = (int)is[2], iw = (int)is[3];
  const int oc = ic / (r * r), oh = ih * r, ow = iw * r;
  int64_t i_index = 0;
  for (int n = 0; n < in; n++)
    for (int c = 0; c < ic; c++)
      for (int h = 0; h < ih; h++)
        for (int w = 0; w < iw; w++) {
          int new_c, new_h, new_w;
          if (dcr_mode) {
            new_c = c % oc;
            new_h = h * r + (c / oc) / r;
            new_w = w * r + ((c / oc) % r);
          } else {
            new_c = c / (r * r);
            new_h = h * r + (c / r) % r;
            new_w = w * r + (c % (r * r)) % r;
          }
          y[(int64_t)n * oc * oh * ow + (int64_t)new_c * oh * ow + (int64_t)new_h * ow + new_w] =
              x[i_index++];
        }
}

/* SwapChannelOpKernel::invoke (core/swap_channel.cpp:21-34): output channel j is input channel
 * order[j], whole frames copied */
void orc_swap_channel_i8(const int8_t *x, int8_t *y, const int64_t *s, const int *order) {
  const int64_t frame = s[2] * s[3], batch = frame * s[1];
  for (int64_t i = 0; i < s[0]; ++i)
    for (int64_t j = 0; j < s[1]; ++j)
      memcpy(y + i * batch + frame * j, x + i * batch + frame * order[j], (size_t)frame);
}

/* ZeroMaskOpKernel::invoke (core/zero_mask.cpp:19-33), INT8: the mask value is 127 */
void orc_zero_mask_i8(const int8_t *x, int8_t *y, int64_t n, int positive) {
  for (int64_t i = 0; i < n; ++i)
    y[i] = x[i] == 0 ? (positive ? 0 : 127) : (positive ? 127 : 0);
}

/* F32ToInt(v, 0) + F32ToInt8 (QuantizationArithmetic.cpp:917-947): nearest, ties to even, on
 * |v|; then saturated */
static int8_t f32_to_int8_nearest_even(float v) {
  float integer;
  const float fraction = modff(fabsf(v), &integer);
  int32_t q = (int32_t)integer;
  if (fraction > 0.5f) q += 1;
  else if (fraction == 0.5f && (q & 1)) q += 1;
  if (v < 0) q = -q;
  return (int8_t)(q > 127 ? 127 : q < -128 ? -128 : q);
}

/* MulConstOpKernel::invoke (core/eltwise.cpp:386-401), INT8: F32ToInt8(x * const_val, 0), then
 * the optional ReLU */
void orc_mul_const_i8(const int8_t *x, int8_t *y, int64_t n, float const_val, int do_relu) {
  for (int64_t i = 0; i < n; ++i) {
    int8_t v = f32_to_int8_nearest_even((float)x[i] * const_val);
    y[i] = do_relu && v < 0 ? 0 : v;
  }
}

/* lrn_int8 (core/lrn.cpp:104-166): squares from a table indexed by the input byte, a sliding
 * sum over local_size channels kept as a running float (add the head, subtract the tail),
 * rescaled to a table index, the power table entry times the input. */
void orc_lrn_i8(const int8_t *x, int8_t *y, int n, int c, int h, int w, int local_size,
                const float *sqr_lut, const float *power_lut, int sq_right_shift, int lrn_right_shift,
                int quant0, int quant1) {
  const int pre_pad = (local_size - 1) / 2, padded_c = c + local_size - 1;
  const int64_t frame = (int64_t)h * w, batch = frame * c;
  float *padded = (float *)calloc((size_t)(padded_c * frame), sizeof(float));
  float *scale = (float *)calloc((size_t)(n * batch), sizeof(float));
  float *square = padded + pre_pad * frame;
  for (int in = 0; in < n; ++in) {
    const int8_t *xn = x + in * batch;
    float *sn = scale + in * batch;
    for (int64_t i = 0; i < batch; ++i) square[i] = sqr_lut[(uint8_t)xn[i]];
    for (int ic = 0; ic < local_size; ++ic)
      for (int64_t i = 0; i < frame; ++i) sn[i] += (float)quant0 * padded[ic * frame + i];
    for (int ic = 1; ic < c; ++ic) {
      memcpy(sn + ic * frame, sn + (ic - 1) * frame, (size_t)frame * sizeof(float));
      for (int64_t i = 0; i < frame; ++i) sn[ic * frame + i] += (float)quant0 * padded[(ic + local_size - 1) * frame + i];
      for (int64_t i = 0; i < frame; ++i) sn[ic * frame + i] += (float)-quant0 * padded[(ic - 1) * frame + i];
    }
  }
  const float sq_scale = 1.0f / (1 << sq_right_shift), lrn_scale = 1.0f / (1 << lrn_right_shift);
  for (int64_t i = 0; i < n * batch; ++i) {
    float t = floorf(scale[i] * sq_scale + 0.5f);
    if (t < 0.0f) t = 0.0f;
    else if (t > 255.0f) t = 255.0f;
    float o = power_lut[(uint8_t)t];
    o *= (float)x[i] * quant1 * lrn_scale;
    o = floorf(o + 0.5f);
    y[i] = (int8_t)(o < -128.0f ? -128.0f : o > 127.0f ? 127.0f : o);
  }
  free(padded);
  free(scale);
}

/* ReduceOpKernel::invoke (core/reduce.cpp:54-117), INT8, kinds 0 mean / 1 sum / 2 max / 3 min over
 * the axes between outer and inner.  In INT8 the mean is a sum too (its 1/axis is folded into the
 * multiplier); the float result is requantised when rshift != 0 or multiplier != 1 and stored
 * as it is otherwise. */
void orc_reduce_i8(int kind, const int8_t *x, int8_t *y, int64_t outer, int64_t axis, int64_t inner,
                   float rshift, float multiplier) {
  for (int64_t o = 0; o < outer; ++o)
    for (int64_t i = 0; i < inner; ++i) {
      float v;
      if (kind <= 1) {
        v = 0.0f;
        for (int64_t a = 0; a < axis; ++a) v += (float)x[o * axis * inner + a * inner + i];
      } else {
        v = (float)x[o * axis * inner + i];
        for (int64_t a = 1; a < axis; ++a) {
          const float t = (float)x[o * axis * inner + a * inner + i];
          if (kind == 2 && t > v) v = t;
          else if (kind == 3 && t < v) v = t;
        }
      }
      if (rshift != 0 || multiplier != 1)
        y[o * inner + i] = orc_apply_mult_rshift_sat8_f(v, (uint32_t)rshift, (uint32_t)multiplier, 0);
      else
        y[o * inner + i] = (int8_t)v;   /* callers only ask for this when v is an int8 value */
    }
}

/* ------------------------------------------------------------------------- */
/* transposed convolution                                                     */
/* ------------------------------------------------------------------------- */
void orc_deconv2d_acc(const int8_t *x, const int8_t *w, int32_t *acc, const orc_conv_desc *d) {
  const int icg = d->ic / d->g, ocg = d->oc / d->g;
  memset(acc, 0, sizeof(int32_t) * (size_t)d->n * d->oc * d->oh * d->ow);
#pragma omp parallel for collapse(2)
  for (int n = 0; n < d->n; ++n)
    for (int oc = 0; oc < d->oc; ++oc) {
      const int g = oc / ocg;
      int32_t *ap = acc + ((size_t)n * d->oc + oc) * d->oh * d->ow;
      for (int c = 0; c < icg; ++c) {
        const int8_t *xp = x + ((size_t)n * d->ic + g * icg + c) * d->ih * d->iw;
        const int8_t *wp = w + ((size_t)oc * icg + c) * d->kh * d->kw;
        for (int ih = 0; ih < d->ih; ++ih)
          for (int iw = 0; iw < d->iw; ++iw) {
            const int32_t xv = xp[ih * d->iw + iw];
            for (int kh = 0; kh < d->kh; ++kh) {
              const int oh = ih * d->sh + kh * d->dh - d->pt;
              if (oh < 0 || oh >= d->oh) continue;
              for (int kw = 0; kw < d->kw; ++kw) {
                const int ow = iw * d->sw + kw * d->dw - d->pl;
                if (ow < 0 || ow >= d->ow) continue;
                ap[oh * d->ow + ow] += xv * (int32_t)wp[kh * d->kw + kw];
              }
            }
          }
      }
    }
}

void orc_deconv2d_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                     const float *multiplier, int8_t *y, const orc_conv_desc *d) {
  const size_t count = (size_t)d->n * d->oc * d->oh * d->ow;
  int32_t *acc = (int32_t *)malloc(count * sizeof(int32_t));
  orc_deconv2d_acc(x, w, acc, d);
  orc_requant_per_channel(acc, y, d->with_bias ? bias : NULL, d->do_relu, d->n, d->oc,
                          (int64_t)d->oh * d->ow, rshift, multiplier);
  free(acc);
}

/* ------------------------------------------------------------------------- */
/* QuantOp                                                                    */
/* ------------------------------------------------------------------------- */

/* QuantizationArithmetic.cpp:873-913, 958-964 */
float orc_bf16(float src, int rounding) {
  uint32_t u;
  memcpy(&u, &src, 4);
  uint16_t h;
  if (rounding) {
    const uint32_t lsb = (u >> 16) & 1;
    u += 0x7fff + lsb;
    h = (uint16_t)(u >> 16);
    if ((h & 0x7f80) == 0x7f80) h = 0x7f7f;
  } else {
    h = (uint16_t)(u >> 16);
  }
  const uint32_t o = (uint32_t)h << 16;
  float dst;
  memcpy(&dst, &o, 4);
  return dst;
}

/* quant.cpp:20-30 */
void orc_quant_f32_to_i8(const float *src, int8_t *dst, size_t count, float scale) {
  for (size_t i = 0; i < count; ++i) {
    const float r = roundf(src[i] * scale);
    int val = r > 127.0f ? 127 : r < -128.0f ? -128 : (int)r;   /* the int conversion of the */
    dst[i] = (int8_t)val;                                       /* reference, made total      */
  }
}

/* quant.cpp:108-116 with zero_point == 0 */
void orc_dequant_i8_to_f32(const int8_t *src, float *dst, size_t count, float scale) {
  const float s = orc_bf16(scale, 1);
  for (size_t i = 0; i < count; ++i)
    dst[i] = orc_bf16(orc_bf16((float)src[i] + 0, 0) * s, 1);
}

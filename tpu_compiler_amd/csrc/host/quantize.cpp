// INT8 quantisation arithmetic on the host; see tpuhip/quantize.hpp.
#include "tpuhip/quantize.hpp"

#include <algorithm>
#include <climits>
#include <cmath>
#include <limits>
#include <stdexcept>

namespace tpuhip {

namespace {

// saturateInt8 / saturateInt32 (QuantizationArithmetic.cpp:301-334, :366-393): floor(f + 0.5)
// evaluated in double, then clamped
int8_t sat8(float f) {
  double q = std::floor((double)f + 0.5);
  if (q > 127) q = 127;
  if (q < -128) q = -128;
  return (int8_t)q;
}

int32_t sat32(float f) {
  if (f > (float)INT_MAX) return INT_MAX;
  if (f < (float)INT_MIN) return INT_MIN;
  return (int32_t)std::floor((double)f + 0.5);
}

float max_quant(int bits) { return (float)((1 << (bits - 1)) - 1); }

}  // namespace

void QuantizeMultiplier(double m, int32_t *quantized_multiplier, int *shift) {
  if (!(m >= 0)) throw std::runtime_error("QuantizeMultiplier: negative multiplier");
  if (m == 0.) {
    *quantized_multiplier = 0;
    *shift = 0;
    return;
  }
  const double q = std::frexp(m, shift);
  int64_t q_fixed = (int64_t)std::round(q * (double)(1ll << 31));
  if (q_fixed == (1ll << 31)) {
    q_fixed /= 2;
    ++*shift;
  }
  if (*shift < -31) {   // everything would be shifted out: flush to zero
    *shift = 0;
    q_fixed = 0;
  }
  *quantized_multiplier = (int32_t)q_fixed;
}

int8_t findRShiftAndMultiplierFromQScale(double qscale, uint32_t *multiplier, bool qdm,
                                         uint32_t max_multiplier) {
  if (qdm) {
    int32_t q = 0;
    int lshift = 0;
    if (qscale >= 1) qscale = 0.999999;
    QuantizeMultiplier(qscale, &q, &lshift);
    if (multiplier) *multiplier = (uint32_t)q;
    return (int8_t)(-lshift);
  }
  if (qscale > max_multiplier) {
    if (multiplier) *multiplier = max_multiplier;
    return 0;
  }
  for (int8_t rshift = 0; rshift < 63; ++rshift) {
    if (qscale * (double)(1ULL << (rshift + 1)) >= (double)max_multiplier) {
      if (multiplier) *multiplier = (uint32_t)(qscale * (double)(1ULL << rshift));
      return rshift;
    }
  }
  if (multiplier) *multiplier = 0;   // qscale too small: shift and multiplier both 0
  return 0;
}

namespace {
// qscale * 2^rshift as the uint32 the reference's `(uint32_t)(qscale * (1 << rshift))` yields.
// That expression is undefined from rshift 31 on (and for products outside uint32), which only
// a degenerate threshold reaches; here those cases give the exact product, clamped.
uint32_t scaled_u32(double qscale, int rshift) {
  const double v = rshift < 31 ? qscale * (1 << rshift) : std::ldexp(qscale, rshift);
  if (!(v > 0)) return 0;
  return v >= 4294967295.0 ? 4294967295u : (uint32_t)v;
}
}  // namespace

uint32_t findMultiplierU32FromQScaleAndRShift(double qscale, int8_t rshift) {
  return scaled_u32(qscale, rshift);
}

int8_t findMultiplierI8FromQScaleAndRShift(double qscale, int8_t rshift) {
  return (int8_t)scaled_u32(qscale, rshift);
}

double findQScaleForFilter(float max_filter, float threshold_y, float threshold_x, int quant_bitwidth) {
  if (threshold_y <= 0) threshold_y = 0.00001;
  // float arithmetic throughout, widened at the end
  return (max_filter * threshold_x) / (max_quant(quant_bitwidth) * threshold_y);
}

double findQScaleForBiasI32(float max_bias, float threshold_y) {
  if (threshold_y <= 0) threshold_y = 0.00001;
  // 0x7fffffff * 0.99 is a double, so the division runs in double on a float numerator
  return (max_bias * 127.0f) / (0x7fffffff * 0.99 * threshold_y);
}

float findMaxWeight(const float *weight, int64_t size) {
  float max_abs = std::fabs(weight[0]);
  for (int64_t i = 0; i < size; ++i)
    if (std::fabs(weight[i]) > max_abs) max_abs = std::fabs(weight[i]);
  return max_abs;
}

int8_t quantizeFilterRShiftAndMultiplier(float w, float threshold_y, float threshold_x, uint32_t rshift,
                                         uint32_t multiplier, bool qdm) {
  if (qdm) rshift += 31;
  const double factor =
      multiplier == 0 ? 0 : (double)(threshold_x / threshold_y) * (double)(1ULL << rshift) / multiplier;
  return sat8((float)(w * factor));
}

int32_t quantizeBiasRShiftAndMultiplier(float w, float threshold_y, uint32_t rshift, uint32_t multiplier,
                                        bool qdm) {
  if (qdm) rshift += 31;
  const double factor =
      multiplier == 0 ? 0 : (double)(128.0f / threshold_y) * (double)(1ULL << rshift) / multiplier;
  return sat32((float)(w * factor));
}

void quantizeWeightInt8Multiplier(const float *filter, const float *bias, int64_t oc, int64_t isz,
                                  float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                                  float *rshift_per_channel, float *multiplier_per_channel,
                                  const std::vector<float> &filter_threshold, int quant_bitwidth) {
  const bool use_threshold = !filter_threshold.empty();
  if (use_threshold && (int64_t)filter_threshold.size() != oc)
    throw std::runtime_error("quantizeWeightInt8Multiplier: one filter threshold per output channel");
  for (int64_t i = 0; i < oc; ++i) {
    const float max_filter = use_threshold ? filter_threshold[i] : findMaxWeight(filter + isz * i, isz);
    double qscale = findQScaleForFilter(max_filter, threshold_y, threshold_x, quant_bitwidth);
    if (qscale >= 1) qscale = 0.999999;   // no left shift on the target: the filter saturates instead
    if (bias) {
      const double qscale_bias = findQScaleForBiasI32(std::fabs(bias[i]), threshold_y);
      if (qscale_bias > qscale && !(qscale_bias >= 1)) qscale = qscale_bias;
    }
    uint32_t multiplier = 0;
    rshift_per_channel[i] = (float)findRShiftAndMultiplierFromQScale(qscale, &multiplier, true);
    multiplier_per_channel[i] = (float)multiplier;
  }
  for (int64_t i = 0; i < oc; ++i) {
    // the float-stored parameters are read back the way the reference passes them on
    const uint32_t rshift = (uint32_t)rshift_per_channel[i], mult = (uint32_t)multiplier_per_channel[i];
    for (int64_t j = 0; j < isz; ++j)
      new_filter[isz * i + j] =
          (float)quantizeFilterRShiftAndMultiplier(filter[isz * i + j], threshold_y, threshold_x, rshift, mult, true);
    if (bias) new_bias[i] = (float)quantizeBiasRShiftAndMultiplier(bias[i], threshold_y, rshift, mult, true);
  }
}

void quantizeWeightInt8ForFC(const float *filter, const float *bias, int64_t batch, int64_t N, int64_t K,
                             float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                             float *rshift_per_batch, float *multiplier_per_batch) {
  const int64_t isz = N * K;
  std::vector<double> qscale(batch);
  for (int64_t i = 0; i < batch; ++i)
    qscale[i] = findQScaleForFilter(findMaxWeight(filter + i * isz, isz), threshold_y, threshold_x);
  if (bias)
    for (int64_t i = 0; i < batch; ++i)
      for (int64_t n = 0; n < N; ++n) {
        const double qb = findQScaleForBiasI32(std::fabs(bias[i * N + n]), threshold_y);
        if (qb > qscale[i]) qscale[i] = qb;
      }
  for (int64_t i = 0; i < batch; ++i) {
    uint32_t multiplier = 0;
    rshift_per_batch[i] = (float)findRShiftAndMultiplierFromQScale(qscale[i], &multiplier, true, 255);
    multiplier_per_batch[i] = (float)multiplier;
  }
  for (int64_t i = 0; i < batch; ++i) {
    const uint32_t rshift = (uint32_t)rshift_per_batch[i], mult = (uint32_t)multiplier_per_batch[i];
    for (int64_t j = 0; j < isz; ++j)
      new_filter[i * isz + j] =
          (float)quantizeFilterRShiftAndMultiplier(filter[i * isz + j], threshold_y, threshold_x, rshift, mult, true);
    if (bias)
      for (int64_t n = 0; n < N; ++n)
        new_bias[i * N + n] =
            (float)quantizeBiasRShiftAndMultiplier(bias[i * N + n], threshold_y, rshift, mult, true);
  }
}

void quantizeRescaleNoWeight(const std::vector<float> &threshold_x, float threshold_y,
                             const std::vector<float> &coeff, int divisor, float *rshift, float *multiplier) {
  const size_t n = threshold_x.size();
  if (!coeff.empty() && coeff.size() != n) throw std::runtime_error("quantizeRescaleNoWeight: one coeff per input");
  std::vector<float> qscale(n);
  for (size_t i = 0; i < n; ++i) {
    qscale[i] = coeff.empty() ? threshold_x[i] / threshold_y : coeff[i] * threshold_x[i] / threshold_y;
    if (qscale[i] < 0) throw std::runtime_error("quantizeRescaleNoWeight: a negative scale has no int8 multiplier");
  }
  if (divisor != 1 && n) qscale[0] = qscale[0] / divisor;
  float max_qscale = 0.0f;
  for (float q : qscale) max_qscale = std::max(max_qscale, q);
  const int8_t r = findRShiftAndMultiplierFromQScale(max_qscale);
  rshift[0] = (float)r;
  for (size_t i = 0; i < n; ++i) multiplier[i] = (float)findMultiplierI8FromQScaleAndRShift(qscale[i], r);
}

void quantizeLeakyRelu(float negative_slope, float threshold_x, float threshold_y, float out[4]) {
  const double qscale_pos = threshold_x / threshold_y;
  if (std::fabs(threshold_x - threshold_y) < 1e-5 * std::min(threshold_x, threshold_y)) {
    out[0] = 0;
    out[1] = 1.0f;   // no positive scale
  } else {
    uint32_t m = 0;
    out[0] = (float)findRShiftAndMultiplierFromQScale(qscale_pos, &m, false);
    out[1] = (float)m;
  }
  const float qscale_neg = std::fabs(qscale_pos * negative_slope);
  uint32_t m = 0;
  out[2] = (float)findRShiftAndMultiplierFromQScale(qscale_neg, &m, false);
  out[3] = (float)m;
}

void quantizeLutTable(LutKind kind, float threshold_x, float threshold_y, float scale, float bias,
                      float coeff, float table256[256]) {
  for (int idx = 0; idx < 256; ++idx) {
    const int8_t in = (int8_t)idx;
    double index = 0, out = 0;
    switch (kind) {
    case LutKind::Pow: {
      const double qscale = 127.0 / threshold_y * std::pow(threshold_x / 127.0, coeff);
      if (coeff < 0 && in == 0) out = 127.0f;
      else if (coeff != (int)coeff && in < 0) out = 0.0f;
      else out = std::pow(in, coeff) * qscale;
      break;
    }
    case LutKind::Sigmoid:
      index = -in * threshold_x / 127.0;
      out = (scale / (1 + std::exp(index)) + bias) * 127.0 / threshold_y;
      break;
    case LutKind::Log:
      index = in * threshold_x / 127.0;
      out = std::log(index) * 127.0 / threshold_y;
      break;
    case LutKind::Swish:
      index = in * threshold_x / 127.0;
      out = index / (1 + std::exp(-index)) * 127.0 / threshold_y;
      break;
    case LutKind::TanH:
      index = in * threshold_x / 127.0;
      out = std::tanh(index) * 127.0 / threshold_y;
      break;
    case LutKind::Elu:
      index = in * threshold_x / 127.0;
      out = ((index >= 0) ? index : (std::exp(index) - 1)) * 127.0 / threshold_y;
      break;
    case LutKind::Exp:
      index = in * threshold_x / 127.0;
      out = (scale * std::exp(index) + bias) * 127.0 / threshold_y;
      break;
    case LutKind::SoftPlus:
      index = in * threshold_x / 127.0;
      out = (scale * logf(expf(index) + 1) + bias) * 127.0 / threshold_y;
      break;
    case LutKind::Mish: {
      // my_mish_activate (lib/Dialect/TPU/Interpreter/NativeCpuImplementation.cpp:527-537):
      // x * tanh(softplus(x)), all in float, tanh as 2 / (1 + exp(-2 s)) - 1
      index = in * threshold_x / 127.0;
      const float xv = (float)index;
      const float sp = logf(expf(xv) + 1);
      out = xv * (2 / (1 + expf(-2 * sp)) - 1) * 127.0 / threshold_y;
      break;
    }
    }
    // INT8(): floor(x + 0.5) clamped (QuantizeInt8.cpp:48-51); a NaN (log of a negative
    // input) passes through both std::min and std::max as their first argument does
    double q = std::floor(out + 0.5);
    q = std::max(std::min(q, 127.0), -128.0);
    table256[idx] = (float)q;
  }
}

}  // namespace tpuhip

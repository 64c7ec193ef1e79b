// C ABI over the host-side quantisation arithmetic: exceptions become status codes.
#include <cstring>
#include <stdexcept>
#include <string>

#include "tpuhip.h"
#include "tpuhip/quantize.hpp"
#include "tpuhip/quantize_pass.hpp"

namespace tpuhip {
int set_error(int status, const char *fmt, ...);
}

using namespace tpuhip;

#define QGUARD(...)                                          \
  try {                                                      \
    __VA_ARGS__;                                             \
  } catch (const std::exception &e) {                        \
    return set_error(TPUHIP_ERR_INVALID, "%s", e.what());    \
  }                                                          \
  return TPUHIP_OK;

extern "C" {

int tpuhip_quantize_multiplier(double multiplier, int32_t *quantized, int *shift) {
  QGUARD({
    if (!quantized || !shift) throw std::runtime_error("quantize_multiplier: NULL argument");
    QuantizeMultiplier(multiplier, quantized, shift);
  })
}

int tpuhip_find_rshift_and_multiplier(double qscale, int qdm, uint32_t max_multiplier, int *rshift,
                                      uint32_t *multiplier) {
  QGUARD({
    if (!rshift || !multiplier) throw std::runtime_error("find_rshift_and_multiplier: NULL argument");
    if (!(qscale >= 0)) throw std::runtime_error("find_rshift_and_multiplier: negative qscale");
    *rshift = findRShiftAndMultiplierFromQScale(qscale, multiplier, qdm != 0, max_multiplier);
  })
}

int tpuhip_quantize_conv_weights(const float *filter, const float *bias, int64_t oc, int64_t isz,
                                 float threshold_y, float threshold_x, const float *filter_threshold,
                                 float *new_filter, float *new_bias, float *rshift, float *multiplier) {
  QGUARD({
    if (!filter || !new_filter || !rshift || !multiplier || (bias && !new_bias) || oc <= 0 || isz <= 0)
      throw std::runtime_error("quantize_conv_weights: bad argument");
    std::vector<float> ft;
    if (filter_threshold) ft.assign(filter_threshold, filter_threshold + oc);
    quantizeWeightInt8Multiplier(filter, bias, oc, isz, threshold_y, threshold_x, new_filter, new_bias, rshift,
                                 multiplier, ft);
  })
}

int tpuhip_quantize_fc_weights(const float *filter, const float *bias, int64_t batch, int64_t n, int64_t k,
                               float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                               float *rshift, float *multiplier) {
  QGUARD({
    if (!filter || !new_filter || !rshift || !multiplier || (bias && !new_bias) || batch <= 0 || n <= 0 || k <= 0)
      throw std::runtime_error("quantize_fc_weights: bad argument");
    quantizeWeightInt8ForFC(filter, bias, batch, n, k, threshold_y, threshold_x, new_filter, new_bias, rshift,
                            multiplier);
  })
}

int tpuhip_quantize_rescale(const float *threshold_x, int n_inputs, float threshold_y, const float *coeff,
                            int divisor, float *rshift, float *multiplier) {
  QGUARD({
    if (!threshold_x || n_inputs <= 0 || !rshift || !multiplier || divisor <= 0)
      throw std::runtime_error("quantize_rescale: bad argument");
    std::vector<float> tx(threshold_x, threshold_x + n_inputs);
    std::vector<float> cf;
    if (coeff) cf.assign(coeff, coeff + n_inputs);
    quantizeRescaleNoWeight(tx, threshold_y, cf, divisor, rshift, multiplier);
  })
}

int tpuhip_quantize_leaky_relu(float negative_slope, float threshold_x, float threshold_y, float *out4) {
  QGUARD({
    if (!out4) throw std::runtime_error("quantize_leaky_relu: NULL argument");
    quantizeLeakyRelu(negative_slope, threshold_x, threshold_y, out4);
  })
}

int tpuhip_quantize_lut_table(int kind, float threshold_x, float threshold_y, float scale, float bias,
                              float coeff, float *table256) {
  QGUARD({
    if (!table256) throw std::runtime_error("quantize_lut_table: NULL argument");
    if (kind < 0 || kind > (int)LutKind::Mish) throw std::runtime_error("quantize_lut_table: unknown kind");
    quantizeLutTable((LutKind)kind, threshold_x, threshold_y, scale, bias, coeff, table256);
  })
}

int tpuhip_quantize_mlir_files(const char *in_mlir, const char *calibration_table, const char *out_mlir,
                               const char *out_weights, char *missing, size_t capacity, size_t *needed) {
  QGUARD({
    if (!in_mlir || !calibration_table || !out_mlir) throw std::runtime_error("quantize_mlir_files: NULL path");
    std::string text;
    for (auto &name : quantizeFiles(in_mlir, calibration_table, out_mlir, out_weights ? out_weights : ""))
      text += name + "\n";
    if (needed) *needed = text.size() + 1;
    if (missing && capacity) {
      const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
      std::memcpy(missing, text.data(), n);
      missing[n] = '\0';
    }
  })
}

}  // extern "C"

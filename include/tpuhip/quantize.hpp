// Host-side INT8 quantisation arithmetic: what the reference's --tpu-quant pass computes
// when it turns an fp32 layer and two calibration thresholds into the float-stored integer
// operands the interpreter's INT8 kernels consume (lib/Dialect/TPU/Quantization/
// QuantizationArithmetic.cpp, QuantizeInt8.cpp).  Every function keeps the reference's mix
// of float and double evaluation, because the integers it produces depend on it.
#pragma once

#include <cstdint>
#include <vector>

namespace tpuhip {

// QuantizationArithmetic.cpp:182-220 (the TensorFlow Lite decomposition): m = q * 2^shift / 2^31
// with q in [2^30, 2^31), or q = 0
void QuantizeMultiplier(double double_multiplier, int32_t *quantized_multiplier, int *shift);

// QuantizationArithmetic.cpp:237-289.  qdm: QuantizeMultiplier form (qscale >= 1 is replaced by
// 0.999999), returns rshift = -shift.  Otherwise the smallest rshift with
// qscale * 2^(rshift+1) >= max_multiplier, multiplier = (uint32)(qscale * 2^rshift).
int8_t findRShiftAndMultiplierFromQScale(double qscale, uint32_t *multiplier = nullptr, bool qdm = false,
                                         uint32_t max_multiplier = 127);
// :291-299
uint32_t findMultiplierU32FromQScaleAndRShift(double qscale, int8_t rshift);
int8_t findMultiplierI8FromQScaleAndRShift(double qscale, int8_t rshift);
// :145-180
double findQScaleForFilter(float max_filter, float threshold_y, float threshold_x, int quant_bitwidth = 8);
double findQScaleForBiasI32(float max_bias, float threshold_y);
// :12-20
float findMaxWeight(const float *weight, int64_t size);
// :437-479
int8_t quantizeFilterRShiftAndMultiplier(float w, float threshold_y, float threshold_x, uint32_t rshift,
                                         uint32_t multiplier, bool qdm);
int32_t quantizeBiasRShiftAndMultiplier(float w, float threshold_y, uint32_t rshift, uint32_t multiplier,
                                        bool qdm);

// Conv / DeConv, per output channel (QuantizationArithmetic.cpp:741-818, called from
// quantizeInt8ConvOps, QuantizeInt8.cpp:56-166).  filter is oc x isz; bias may be null.
// filter_threshold: empty, or one max |w| per channel to use instead of the measured one.
void quantizeWeightInt8Multiplier(const float *filter, const float *bias, int64_t oc, int64_t isz,
                                  float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                                  float *rshift_per_channel, float *multiplier_per_channel,
                                  const std::vector<float> &filter_threshold = {}, int quant_bitwidth = 8);

// FullyConnected, one rshift / multiplier per batch (QuantizationArithmetic.cpp:630-690)
void quantizeWeightInt8ForFC(const float *filter, const float *bias, int64_t batch, int64_t N, int64_t K,
                             float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                             float *rshift_per_batch, float *multiplier_per_batch);

// Ops without weights that rescale their inputs (eltwise add / max / min, concat-like, avg
// pool): one rshift and one int8 multiplier per input (quantizeInt8RescaleNoWeightOps,
// QuantizeInt8.cpp:669-854).  coeff: empty or one factor per input (eltwise add);
// divisor: kh * kw for an average pool, the reduced size for a mean, else 1.
void quantizeRescaleNoWeight(const std::vector<float> &threshold_x, float threshold_y,
                             const std::vector<float> &coeff, int divisor, float *rshift, float *multiplier);

// LeakyRelu (quantizeInt8LeakyReluOps, QuantizeInt8.cpp:349-429): out[0..3] = rshift_pos,
// multiplier_pos, rshift_neg, multiplier_neg
void quantizeLeakyRelu(float negative_slope, float threshold_x, float threshold_y, float out[4]);

// 256-entry tables of the table-lookup activations (quantizeInt8LutOps, QuantizeInt8.cpp:531-621),
// index = the two's-complement byte of the int8 input.  scale / bias: the op attributes of
// sigmoid, exp and softplus (1 and 0 when the op has none); coeff: the exponent of pow.
enum class LutKind { Sigmoid, TanH, Exp, Elu, Swish, SoftPlus, Log, Pow, Mish };
void quantizeLutTable(LutKind kind, float threshold_x, float threshold_y, float scale, float bias,
                      float coeff, float table256[256]);

}  // namespace tpuhip

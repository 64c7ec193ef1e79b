/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement (plain C) of the arithmetic the
 * tpuc-interpreter performs on its INT8 path.  It is the checker the HIP
 * kernels are compared against; nothing that ships may link or call it.
 *
 * Tensors are NCHW (W fastest) like the reference's.  Activations and
 * weights are int8; every quantisation parameter is passed the way the
 * reference stores it -- as a float holding an integer -- so that the
 * float -> uint32 -> int32 conversions of the reference are reproduced here
 * and not by the caller.
 *
 * Each function names the reference lines it follows (paths relative to the
 * reference tree).
 *
 * Parity status: the reference has no stored expected outputs for this path
 * and cannot be built offline (needs MLIR and MKL-DNN 1.0.2).  Every function
 * below is pinned by closed forms / brute force / library cross-checks in
 * tests/; the one behaviour that nothing pins is MKL-DNN's fp32 accumulation
 * order when partial sums exceed 2^24 ("parity unpinned"); orc_conv2d_guard
 * and orc_fc_guard report when an input leaves the exact domain.
 */
#ifndef TPU_ORACLE_H
#define TPU_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- scalar arithmetic: lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp ---- */

/* :501-509 */
int32_t orc_srdhm(int32_t a, int32_t b);
/* :487-499.  exponent outside [0,31] is outside the reference's assert; returns x. */
int32_t orc_rdbp(int32_t x, int exponent);
/* :301-334 (the "#elif 1" branch: floor(f + 0.5), clamp) */
int8_t orc_saturate_int8(float f);
/* :481-483 */
int8_t orc_apply_rshift_sat8(float v, uint32_t rshift);
/* :518-528 (float overload) */
int8_t orc_apply_mult_rshift_sat8_f(float v, uint32_t rshift, uint32_t multiplier, int qdm);
/* :530-539 (int32 overload) */
int8_t orc_apply_mult_rshift_sat8_i(int32_t v, uint32_t rshift, uint32_t multiplier, int qdm);
/* the implicit float -> uint32_t conversion at :849-863 as x86-64 gcc emits it
 * (cvttss2si to 64 bit, low 32 bits kept) */
uint32_t orc_f2u32(float f);

/* ---- convolution: lib/Dialect/TPU/Interpreter/core/conv.cpp:11-104 ---- */
typedef struct {
  int n, ic, ih, iw;
  int oc, oh, ow;
  int g;
  int kh, kw;
  int sh, sw;
  int pt, pb, pl, pr;
  int dh, dw;
  int ins_h, ins_w; /* zeros inserted between input rows / columns (conv.cpp:66-77) */
  int do_relu;
  int with_bias;
} orc_conv_desc;

/* Integer cross-correlation, zero padding (include/tpuc/NativeCpuImplementation.h:11-102
 * restated in int32).  x: n*ic*ih*iw, w: oc*(ic/g)*kh*kw, acc: n*oc*oh*ow. */
void orc_conv2d_acc(const int8_t *x, const int8_t *w, int32_t *acc, const orc_conv_desc *d);
/* max over outputs of sum_k |x_k * w_k|: fp32 accumulation is order-independent
 * and equal to the int32 sum whenever this is < 2^24. */
int64_t orc_conv2d_guard(const int8_t *x, const int8_t *w, const orc_conv_desc *d);
/* The same contraction done the reference's way: float-stored operands, fp32
 * accumulate (one fixed order).  Used to show fp32 == int32 under the guard. */
void orc_conv2d_acc_f32(const float *x, const float *w, float *acc, const orc_conv_desc *d);
/* QuantizationArithmetic.cpp:849-871, input = int32 accumulators.
 * bias may be NULL. */
void orc_requant_per_channel(const int32_t *acc, int8_t *y, const float *bias, int do_relu,
                             int64_t on, int64_t oc, int64_t isz, const float *rshift,
                             const float *multiplier);
/* whole op: conv.cpp:80-104 (INT8 branch).  bias/rshift/multiplier hold oc floats. */
void orc_conv2d_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                   const float *multiplier, int8_t *y, const orc_conv_desc *d);

/* ---- transposed convolution: core/deconv.cpp:56-73 over MKLDeconv
 * (NativeCpuImplementation.h:194-280: deconvolution_direct, filter oihw / goihw with o = this
 * op's output channels).  Every input pixel scatters into the outputs
 * (ih*sh + kh*dh - pt, iw*sw + kw*dw - pl); then the conv's per-channel epilogue.
 * d uses the deconvolution's own stride / padding / dilation; ins_* are ignored. ---- */
void orc_deconv2d_acc(const int8_t *x, const int8_t *w, int32_t *acc, const orc_conv_desc *d);
void orc_deconv2d_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                     const float *multiplier, int8_t *y, const orc_conv_desc *d);

/* ---- fully connected: core/fullyconnected.cpp:44-91 (no transposes), one
 * rshift / multiplier per batch matmul.  x: batch*m*k, w: batch*n*k,
 * bias: batch*n or NULL, y: batch*m*n ---- */
void orc_fc_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
               const float *multiplier, int8_t *y, int batch, int m, int k, int n, int do_relu);
void orc_fc_batched_i8(const int8_t *x, const int8_t *w, const float *bias, const float *rshift,
                       const float *multiplier, int8_t *y, int batch_high, int batch_low, int m,
                       int k, int n, int ltrans, int otrans, int do_relu);
int64_t orc_fc_guard(const int8_t *x, const int8_t *w, const float *bias, int batch, int m, int k,
                     int n);

/* ---- eltwise add: core/eltwise.cpp:52-85 ---- */
void orc_eltwise_add_i8(const int8_t *const *xs, int nin, const float *multiplier,
                        const float *rshift, int do_relu, int8_t *y, size_t count);

/* ---- two-input elementwise ops with broadcasting ----
 * core/eltwise.cpp:143-189 (Max), 233-279 (Min), 324-347 (Mul) and core/broadcast.cpp:45-154
 * (BroadcastAdd / Mul / Sub).  Every dimension of an operand equals the output's or is 1.
 * add/sub/max/min: each input times (int8_t)multiplier[i] in float, combined, ReLU, then
 * v / 2^rshift and floor(. + 0.5), saturate.  mul: product, ReLU, qdm requant with
 * (uint32)rshift, (uint32)multiplier[0].  Returns -1 for the one case with no int8 meaning:
 * an eltwise mul with rshift == 0 and multiplier == 0 (the reference leaves the raw product). */
enum { ORC_BIN_ADD = 0, ORC_BIN_SUB = 1, ORC_BIN_MAX = 2, ORC_BIN_MIN = 3, ORC_BIN_MUL = 4 };
typedef struct {
  int op;
  int n, c, h, w;       /* output */
  int n0, c0, h0, w0;   /* operand 0 */
  int n1, c1, h1, w1;   /* operand 1 */
  int do_relu;
} orc_binary_desc;
int orc_binary_i8(const int8_t *x0, const int8_t *x1, int8_t *y, const orc_binary_desc *d,
                  const float *multiplier, float rshift);

/* ---- pooling: core/pooling.cpp:89-160 (normal path only) ---- */
typedef struct {
  int n, c, ih, iw, oh, ow, kh, kw, sh, sw, pt, pb, pl, pr;
} orc_pool_desc;
void orc_pool_max_i8(const int8_t *x, int8_t *y, const orc_pool_desc *d);
void orc_pool_avg_i8(const int8_t *x, int8_t *y, const orc_pool_desc *d, float rshift,
                     float multiplier);

/* ---- activations: core/activation.cpp ---- */
/* :126-153 */
void orc_leaky_relu_i8(const int8_t *x, int8_t *y, size_t count, float rshift_pos,
                       float multiplier_pos, float rshift_neg, float multiplier_neg);
/* :185-224 PRelu: x > 0 -> non-qdm (x * multiplier_pos) / 2^rshift_pos; else slope[c] * x then
 * / 2^rshift_neg; both floor(. + 0.5), saturate.  slope holds c floats. */
void orc_prelu_i8(const int8_t *x, int8_t *y, int n, int c, int hw, const float *slope,
                  float rshift_pos, float multiplier_pos, float rshift_neg);
/* :47-53 and siblings: y = table[(unsigned char)x]; table holds 256 floats */
void orc_scale_lut_u8(const uint8_t *x, int8_t *y, int n, int c, int hw, const float *table);
void orc_lut_i8(const int8_t *x, int8_t *y, size_t count, const float *table256);
/* :155-164 + core/internal.cpp:13-18 */
void orc_relu_i8(const int8_t *x, int8_t *y, size_t count);
/* core/clip.cpp:29-40 */
void orc_clip_i8(const int8_t *x, int8_t *y, size_t count, float min, float max, float rshift,
                 float multiplier);

/* ---- data movement ---- */
/* core/upsample.cpp:20-41 */
void orc_upsample_i8(const int8_t *x, int8_t *y, int n, int c, int ih, int iw, int scale_h,
                     int scale_w);
/* core/concat.cpp:34-90.  shapes: nin*ndim int64 (row per input).  rshift /
 * multiplier NULL when the op carries none. */
void orc_concat_i8(const int8_t *const *xs, int nin, const int64_t *shapes, int ndim, int axis,
                   const float *rshift, const float *multiplier, int do_relu, int8_t *y);

/* ---- QuantOp at the graph edges: core/quant.cpp:9-32 (fp32 -> int8 right after an input:
 * round(src * scale), half away from zero, clamped; zero_point is 0, :138) and :108-124
 * (int8 -> fp32, always the TPU-aligned form: BF16(BF16(src) * BF16(scale)) with the
 * round-to-nearest-even BF16 of QuantizationArithmetic.cpp:873-913, infinity clipped). ---- */
void orc_quant_f32_to_i8(const float *src, int8_t *dst, size_t count, float scale);
void orc_dequant_i8_to_f32(const int8_t *src, float *dst, size_t count, float scale);
float orc_bf16(float src, int rounding);

/* ---- pure data movement (no INT8-specific branch in the reference), 4-d shapes ---- */
/* core/pad.cpp:62-112 (constant mode; negative pads cut) and :7-60 (edge mode, h/w only).
 * pads = {n,c,h,w begin, n,c,h,w end}.  The reference never reads const_val: constant
 * padding is the zero of the freshly created result tensor. */
void orc_pad_i8(const int8_t *x, int8_t *y, const int64_t *ishape, const int *pads, int edge_mode);
/* core/crop.cpp:44-92: y[o] = x[o * steps + offset] per dimension */
void orc_crop_i8(const int8_t *x, int8_t *y, const int64_t *ishape, const int64_t *oshape,
                 const int *offset, const int *steps);
/* core/permute.cpp:8-33: output dimension k is input dimension order[k] */
void orc_permute_i8(const int8_t *x, int8_t *y, const int64_t *ishape, const int *order);
/* core/reorg.cpp:20-42 */
void orc_reorg_i8(const int8_t *x, int8_t *y, const int64_t *ishape, int stride);
/* core/tile.cpp:24-42: the block from `axis` on is repeated `tiles` times */
void orc_tile_i8(const int8_t *x, int8_t *y, const int64_t *ishape, int axis, int tiles);
/* core/reverse.cpp:19-42 */
void orc_reverse_i8(const int8_t *x, int8_t *y, const int64_t *shape, int axis);
/* core/shuffle_channel.cpp:21-48 */
void orc_shuffle_channel_i8(const int8_t *x, int8_t *y, const int64_t *shape, int group);
/* core/depthtospace.cpp:8-58 (pixelshuffle), dcr_mode as in :60 */
/* core/swap_channel.cpp:21-34, core/zero_mask.cpp:19-33, core/eltwise.cpp:386-401 (INT8 branches) */
void orc_swap_channel_i8(const int8_t *x, int8_t *y, const int64_t *shape, const int *order);
void orc_dilate_i8(const int8_t *x, int8_t *y, const int64_t *shape, int ins_h, int ins_w, int fill);
void orc_reflection_pad_i8(const int8_t *x, int8_t *y, const int64_t *shape, int pad_l, int pad_r);
void orc_zero_mask_i8(const int8_t *x, int8_t *y, int64_t n, int positive);
void orc_mul_const_i8(const int8_t *x, int8_t *y, int64_t n, float const_val, int do_relu);
/* core/lrn.cpp:104-166, INT8 */
void orc_lrn_i8(const int8_t *x, int8_t *y, int n, int c, int h, int w, int local_size,
                const float *sqr_lut, const float *power_lut, int sq_right_shift, int lrn_right_shift,
                int quant0, int quant1);
/* core/reduce.cpp:54-117, INT8; kind 0 mean, 1 sum, 2 max, 3 min */
void orc_reduce_i8(int kind, const int8_t *x, int8_t *y, int64_t outer, int64_t axis, int64_t inner,
                   float rshift, float multiplier);
void orc_depth_to_space_i8(const int8_t *x, int8_t *y, const int64_t *ishape, int upscale,
                           int dcr_mode);

#ifdef __cplusplus
}
#endif
#endif

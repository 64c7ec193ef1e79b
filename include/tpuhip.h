/*
 * tpuhip -- C ABI of the MI355X (gfx950) INT8 kernels that stand in for the
 * tpuc-interpreter's CPU op kernels.  Plain pointers and sizes only.
 *
 * Every entry point returns 0 on success or a tpuhip_status; the message of
 * the last failure on the calling thread is available from
 * tpuhip_last_error().  (The reference aborts through llvm_unreachable /
 * assert instead: lib/Dialect/TPU/Interpreter/MlirModuleInterpreter.cpp:339-344.)
 *
 * Device tensors are int8, channels-last: element (n, h, w, c) of a tensor
 * with channel stride cs lives at byte ((n*H + h)*W + w)*cs + c.  cs is a
 * multiple of 16 and the bytes c..cs-1 of every pixel are zero; every kernel
 * keeps that invariant.  One exception: a tensor of at most 4 channels that only
 * stem convs read may lie at cs = 4 (tpuhip_conv2d_set_input_stride; the layout
 * conversions below take cs = 4 as well).
 * The reference's NCHW float tensors (include/tpuc/Interpreter/cpukernel.h:15-78)
 * are converted at the edge by the tpuhip_*_nchw_* entry points.
 *
 * A context owns one HIP stream; all work of a context is issued to it in call
 * order and is asynchronous until tpuhip_sync().  Calls on one context must be
 * serialised by the caller (the reference is single-threaded as well).
 */
#ifndef TPUHIP_H
#define TPUHIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum {
  TPUHIP_OK = 0,
  TPUHIP_ERR_INVALID = 1,     /* bad argument / shape the kernels cannot take */
  TPUHIP_ERR_HIP = 2,         /* a HIP runtime call failed */
  TPUHIP_ERR_NOMEM = 3,
  TPUHIP_ERR_UNSUPPORTED = 4
} tpuhip_status;

typedef struct tpuhip_ctx tpuhip_ctx;

/* ---- context, memory -------------------------------------------------- */

/* Replaces the construction of MlirModuleInterpreter (include/tpuc/MlirModuleInterpreter.h:34-37):
 * one context per interpreter instance. */
int tpuhip_ctx_create(int device, tpuhip_ctx **out);
/* Same, but work is issued to an existing hipStream_t owned by the caller. */
int tpuhip_ctx_create_on_stream(int device, void *hip_stream, tpuhip_ctx **out);
int tpuhip_ctx_destroy(tpuhip_ctx *ctx);
void *tpuhip_ctx_stream(tpuhip_ctx *ctx);
/* When enabled (the default; TPUHIP_AUTOTUNE=0 in the environment disables it) a
 * dense conv times its tile variants on first use and keeps the fastest.  Every
 * variant produces the same bytes.  The first use of a layer is then not
 * capturable into a HIP graph. */
int tpuhip_ctx_set_autotune(tpuhip_ctx *ctx, int enable);
const char *tpuhip_last_error(void);
const char *tpuhip_version(void);

/* Replaces TensorData's std::vector<float> storage (cpukernel.h:15-24). */
int tpuhip_malloc(tpuhip_ctx *ctx, size_t bytes, void **dptr);
int tpuhip_free(tpuhip_ctx *ctx, void *dptr);
/* Page-locked host memory for staging tensors that cross the host boundary (set_tensor /
 * get_tensor of the module, which hold the reference's std::vector<float> contract,
 * MlirModuleInterpreter.h:47-52): copies from it run as DMA instead of through the driver's
 * bounce buffers.  No counterpart in the reference (its tensors never leave host memory). */
int tpuhip_host_malloc(tpuhip_ctx *ctx, size_t bytes, void **hptr);
int tpuhip_host_free(tpuhip_ctx *ctx, void *hptr);
int tpuhip_memset(tpuhip_ctx *ctx, void *dptr, int value, size_t bytes);
/* Free and total device memory as the HIP runtime this library is linked with reports them (a process
 * may hold a second copy of the runtime, e.g. the one a Python package bundles, which sees other
 * figures or no device).  No counterpart in the reference. */
int tpuhip_mem_info(tpuhip_ctx *ctx, size_t *free_bytes, size_t *total_bytes);
int tpuhip_upload(tpuhip_ctx *ctx, void *dst_dev, const void *src_host, size_t bytes);
int tpuhip_download(tpuhip_ctx *ctx, void *dst_host, const void *src_dev, size_t bytes);
int tpuhip_sync(tpuhip_ctx *ctx);

/* HIP events on the context's stream, for timing what was issued between two
 * records (the reference has no counterpart: its Timer is commented out,
 * bindings/python/pytuner.cpp:55-73). */
int tpuhip_event_create(tpuhip_ctx *ctx, void **event);
int tpuhip_event_destroy(tpuhip_ctx *ctx, void *event);
int tpuhip_event_record(tpuhip_ctx *ctx, void *event);
/* waits for 'stop', then returns the milliseconds between the two records */
int tpuhip_event_elapsed_ms(tpuhip_ctx *ctx, void *start, void *stop, float *ms);

/* While a pair of events is set, every kernel the context launches records its own
 * begin and end of execution into them (the last launch wins), so
 * tpuhip_event_elapsed_ms(start, stop) is that kernel's duration without the gaps
 * around it.  Pass NULL, NULL to switch back. */
int tpuhip_ctx_set_kernel_events(tpuhip_ctx *ctx, void *start, void *stop);

/* channel stride the library uses for a tensor with c channels */
int tpuhip_channel_stride(int c);

/* ---- layout / storage conversion at the API edge ----------------------- */

/* int8 NCHW (dense, device) <-> int8 channels-last with stride cs (device) */
int tpuhip_nchw_to_nhwc_i8(tpuhip_ctx *ctx, const void *src_nchw, void *dst_nhwc, int n, int c,
                           int h, int w, int cs);
int tpuhip_nhwc_to_nchw_i8(tpuhip_ctx *ctx, const void *src_nhwc, void *dst_nchw, int n, int c,
                           int h, int w, int cs);
/* float-stored NCHW (device) <-> int8 channels-last: the float <-> int8 edge of
 * InputOpKernel::set_tensor (core/input.cpp:16-24) and CPUOpKernel::get_tensor
 * (cpukernel.h:124-128).  Floats must hold integers in [-128,127]. */
int tpuhip_nchw_f32_to_nhwc_i8(tpuhip_ctx *ctx, const void *src_f32, void *dst_nhwc, int n, int c,
                               int h, int w, int cs);
int tpuhip_nhwc_i8_to_nchw_f32(tpuhip_ctx *ctx, const void *src_nhwc, void *dst_f32, int n, int c,
                               int h, int w, int cs);

/* ---- Conv2D (dense, grouped, depthwise) -------------------------------- */

/* Field meaning follows parseConvParam (lib/Dialect/TPU/IR/TPUOperationSupport.cpp:366-428). */
typedef struct {
  int n, ic, ih, iw;
  int oc, oh, ow;
  int g;
  int kh, kw;
  int sh, sw;
  int pt, pb, pl, pr;
  int dh, dw;
  int ins_h, ins_w;
  int do_relu;
  int with_bias;
  int x_cs, y_cs;    /* channel strides of input / output */
  int relu_first;    /* 0: ReLU after saturation (conv); 1: ReLU on the sum before requant (FC) */
  int algo;          /* 0 auto, 1 direct (one thread per output), 2 MFMA implicit GEMM, 3 depthwise
                        (one diagonal MFMA per tap), 4 depthwise with per-byte dot products,
                        5 stem (at most 4 input and 64 output channels: input rows staged once in
                        LDS, one MFMA K step per filter row), 16 + t: MFMA tile variant t */
} tpuhip_conv_desc;

typedef struct tpuhip_conv_weights tpuhip_conv_weights;

/* Replaces Conv2DOpKernel's constructor + MKLConv::setup (core/conv.cpp:11-78,
 * include/tpuc/NativeCpuImplementation.h:18-56): takes host OIHW int8 filter
 * (G x OC/G x IC/G x KH x KW for groups), int32 bias (may be NULL), and the
 * per-channel int32 multiplier / rshift the epilogue uses, and stores them on
 * the device in the layout the chosen kernel reads.  rshift must be in [0,31]. */
int tpuhip_conv2d_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *desc, const int8_t *filter_oihw,
                          const int32_t *bias, const int32_t *multiplier, const int32_t *rshift,
                          tpuhip_conv_weights **out);
int tpuhip_conv2d_weights_destroy(tpuhip_ctx *ctx, tpuhip_conv_weights *w);
/* Replaces Conv2DOpKernel::invoke, INT8 branch: MKLConv::run +
 * quantizeActivationInt8PerChannelMultiplierAndRShift (core/conv.cpp:80-104,
 * lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp:849-871). */
int tpuhip_conv2d_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y);
/* Conv2D with an EltwiseAdd folded into its epilogue (a dense conv on the MFMA path
 * only): besides y (written unless y is NULL) the call writes
 *   add_out = sat8(floor(relu?(add_src * m_src + y * m_conv) / 2^rshift + 0.5)),
 * i.e. EltwiseAddOpKernel::i8_invoke (core/eltwise.cpp:52-85) applied to
 * (add_src, y).  add_src / add_out have the shape and channel stride of y.
 * The results equal running the two ops one after the other. */
typedef struct {
  int enable;
  int m_src, m_conv;   /* int8 multipliers of add_src and of the conv result */
  int rshift;          /* 0..30 */
  int do_relu;
} tpuhip_fused_add;
int tpuhip_conv2d_add_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
                         const void *add_src, void *add_out, const tpuhip_fused_add *f);
/* General form of what can ride in a dense conv's epilogue, in this order:
 *   z0 = conv result                          -> y        (if not NULL)
 *   z1 = lut ? lut[(uint8_t)z0] : z0          -> lut_out  (if not NULL)   [LutOpKernel and its
 *        subclasses: core/activation.cpp:47-53, 126-153; core/clip.cpp:29-40]
 *   z2 = add.enable ? EltwiseAdd(add_src, z1) -> add_out                  [core/eltwise.cpp:52-85]
 * lut is a HOST table of 256 int8 entries indexed by the two's-complement byte of the input (passed by
 * value to the kernel).  Only the LDS kernel variants can apply a table; the variant is chosen among them
 * when the first use of the layer is this call. */
typedef struct tpuhip_conv_post {
  const int8_t *lut;
  void *lut_out;
  tpuhip_fused_add add;
  const void *add_src;
  void *add_out;
  /* a max pool (PoolingOpKernel::invoke, core/pooling.cpp, INT8 max branch) over the conv result, run in
   * the conv's launch: pool_out receives what tpuhip_pool_max_i8 would compute from y; y may then be
   * NULL (the conv result itself is not written).  Only where tpuhip_conv2d_can_fuse_pool says so; takes
   * no table and no add.  NULL: no pool. */
  const struct tpuhip_pool_desc *pool;
  void *pool_out;
} tpuhip_conv_post;
int tpuhip_conv2d_post_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y,
                          const tpuhip_conv_post *post);
/* Two Conv2DOpKernel::invoke calls as one launch: two dense convs that read the same input
 * through the same window geometry (kernel, stride, padding, dilation), e.g. the projection
 * shortcut and the first 1x1 conv of a residual block.  Their filters are stacked along the
 * output channels; every output tile goes to the result it belongs to, with that conv's own
 * channel stride and ReLU.  The first conv needs a multiple of 128 output channels.  Results are
 * those of two tpuhip_conv2d_i8 calls.  No counterpart in the reference (one kernel per op). */
int tpuhip_conv2d_prepack_pair(tpuhip_ctx *ctx, const tpuhip_conv_desc *desc_a, const tpuhip_conv_desc *desc_b,
                               const int8_t *filter_a, const int32_t *bias_a, const int32_t *multiplier_a,
                               const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                               const int32_t *multiplier_b, const int32_t *rshift_b,
                               tpuhip_conv_weights **out);
int tpuhip_conv2d_pair_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y_a, void *y_b);
/* Two Conv2DOpKernel::invoke calls (core/conv.cpp:80-104), with an EltwiseAddOpKernel::i8_invoke
 * (core/eltwise.cpp:52-85) between them, as one launch: conv A and conv B are unpadded 1x1 / stride 1
 * convs, B reads what A produced -- or, with an add, the sum of A's result and add_src.  In a residual
 * network: the 1x1 expansion + add that closes a bottleneck block and the 1x1 reduction that opens the
 * next; the sum is written once and not read back.  Shapes covered: A 33..64 -> 256 channels with
 * B 256 -> 64, A 65..128 -> 512 with B 512 -> 128, dense channel strides, right shifts of at least 1
 * and sums that cannot overflow the rounding (tpuhip_conv2d_can_chain answers for the shapes; prepack
 * returns TPUHIP_ERR_UNSUPPORTED otherwise).  y_a (A's own result) and add_out may be NULL: not
 * written.  Results are those of the separate calls.  No counterpart in the reference (one kernel per
 * op). */
typedef struct tpuhip_conv_chain tpuhip_conv_chain;
int tpuhip_conv2d_can_chain(const tpuhip_conv_desc *desc_a, const tpuhip_conv_desc *desc_b);
/* A second kind of chain: conv A a depthwise conv (g == ic == oc, at most 3 x 3 taps, any stride,
 * padding and dilation; core/conv.cpp:11-78, the g != 1 branch), conv B the unpadded 1x1 / stride 1 conv
 * of at most 384 output channels that reads A's result -- the depthwise + projection half of an
 * inverted-residual block.  A 256-entry table (LutOpKernel: core/activation.cpp:47-53,
 * core/clip.cpp:29-40) may ride behind A and an EltwiseAdd (core/eltwise.cpp:52-85) behind B; A's
 * result, the widest tensor of the block, stays on chip unless the caller keeps it.
 * tpuhip_conv2d_chain_kind: 0 = the two convs do not chain, 1 = two pointwise convs (an add behind A),
 * 2 = depthwise then pointwise (a table behind A, an add behind B).  tpuhip_conv2d_can_chain answers
 * kind != 0 and tpuhip_conv2d_chain_prepack packs either kind. */
int tpuhip_conv2d_chain_kind(const tpuhip_conv_desc *desc_a, const tpuhip_conv_desc *desc_b);
int tpuhip_conv2d_chain_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *desc_a, const tpuhip_conv_desc *desc_b,
                                const int8_t *filter_a, const int32_t *bias_a, const int32_t *multiplier_a,
                                const int32_t *rshift_a, const int8_t *filter_b, const int32_t *bias_b,
                                const int32_t *multiplier_b, const int32_t *rshift_b, tpuhip_conv_chain **out);
int tpuhip_conv2d_chain_destroy(tpuhip_ctx *ctx, tpuhip_conv_chain *chain);
/* f == NULL or f->enable == 0: no add, B reads A's result (add_src / add_out ignored) */
int tpuhip_conv2d_chain_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *chain, const void *x, void *y_a,
                           const void *add_src, void *add_out, const tpuhip_fused_add *f, void *y_b);
/* The general call: post_a / post_b (either may be NULL) say what rides behind conv A and conv B, with
 * tpuhip_conv_post's meaning (no pool); y_a, y_b and the outputs inside the posts may be NULL where the
 * caller does not keep a tensor, as long as something of B's is written.  A chain refuses, with an error,
 * the fused work its kind does not take. */
int tpuhip_conv2d_chain_post_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *chain, const void *x, void *y_a,
                                const tpuhip_conv_post *post_a, void *y_b, const tpuhip_conv_post *post_b);
/* A chain of three: the 1x1 expansion (at most 160 input channels), the depthwise conv (at most 3 x 3 taps,
 * any stride, padding and dilation) and the 1x1 projection (at most 384 output channels) of an
 * inverted-residual block, with the block's EltwiseAdd behind the projection (post->add; no table, no
 * pool) -- Conv2DOpKernel::invoke three times (core/conv.cpp:11-104) and EltwiseAddOpKernel::i8_invoke
 * (core/eltwise.cpp:52-85) as one launch.  Neither expanded tensor is written: the call is for graphs in
 * which nothing else reads them.  tpuhip_conv2d_can_chain3 answers for the shapes; prepack returns
 * TPUHIP_ERR_UNSUPPORTED for shapes not covered, a right shift of 0 or sums that could overflow the
 * rounding.  y may be NULL when only the sum is wanted.  The handle is destroyed with
 * tpuhip_conv2d_chain_destroy.  No counterpart in the reference (one kernel per op). */
typedef struct {
  const int8_t *filter;       /* OIHW */
  const int32_t *bias;        /* may be NULL */
  const int32_t *multiplier, *rshift;
} tpuhip_chain_conv;
int tpuhip_conv2d_can_chain3(const tpuhip_conv_desc *expand, const tpuhip_conv_desc *depthwise,
                             const tpuhip_conv_desc *project);
int tpuhip_conv2d_chain3_prepack(tpuhip_ctx *ctx, const tpuhip_conv_desc *expand, const tpuhip_conv_desc *depthwise,
                                 const tpuhip_conv_desc *project, const tpuhip_chain_conv *expand_w,
                                 const tpuhip_chain_conv *depthwise_w, const tpuhip_chain_conv *project_w,
                                 tpuhip_conv_chain **out);
int tpuhip_conv2d_chain3_i8(tpuhip_ctx *ctx, const tpuhip_conv_chain *chain, const void *x, void *y,
                            const tpuhip_conv_post *post);
const char *tpuhip_conv2d_chain_name(const tpuhip_conv_chain *chain);
/* name of chain kernel variant `variant`, NULL past the last one */
const char *tpuhip_conv2d_chain_variant_name(int variant);
/* The channel stride of the input a packed conv will be run on, changed after packing.  4 (one dword per
 * pixel) is taken only by a conv on the stem path -- g == 1, at most 4 input channels, at most 64 output
 * channels, kh <= 7, kw <= 8, stride_w <= 2, which reads a pixel as one dword anyway (TPUHIP_ERR_UNSUPPORTED
 * otherwise): a 3-channel image then occupies a quarter of the bytes of the 16-byte stride and the stem
 * fetches a quarter.  The interpreter lays a graph input out that way when stem convs are its only readers.
 * No counterpart in the reference (its tensors are dense float NCHW, cpukernel.h:15-24). */
int tpuhip_conv2d_set_input_stride(tpuhip_conv_weights *w, int x_cs);
/* name of the kernel variant a prepacked conv dispatches to (for profiling) */
const char *tpuhip_conv2d_algo_name(const tpuhip_conv_weights *w);
/* name of MFMA tile variant `tile` (selected with algo = 16 + tile), NULL past the last one */
const char *tpuhip_conv2d_tile_name(int tile);
/* 1 when tpuhip_conv2d_post_i8 can apply a 256-entry table in this packed conv's epilogue: depthwise
 * and stem kernels always, a dense conv unless its tile variant is fixed (asked for by the caller, or
 * already chosen by timing) to one without a table stage.  The interpreter asks before it folds a
 * table op into its producer (the decision MlirModuleInterpreter.cpp:165-344 never has to make: the
 * reference runs every op as its own kernel). */
int tpuhip_conv2d_can_fuse_table(const tpuhip_conv_weights *w);
/* 1 when tpuhip_conv2d_post_i8 can run this max pool in the packed conv's launch: a stem conv (at most 4
 * input channels, 33..64 output channels, 4..7 filter rows, stride_w <= 2) with ReLU and overflow-free
 * requantisation, a 3x3 / stride 2 pool with top / left padding of at most 1 over exactly the conv's
 * result.  The conv + ReLU + pool head of the ImageNet networks then costs one launch and the conv
 * result stays on chip.  No counterpart in the reference (one kernel per op). */
int tpuhip_conv2d_can_fuse_pool(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const struct tpuhip_pool_desc *pool);

/* ---- FullyConnected ----------------------------------------------------- */

/* Replaces FullyConnectedOpKernel::invoke, INT8 branch (core/fullyconnected.cpp:44-91)
 * for batch == 1, no transposes: y[m][n] = qdm(relu?(sum_k x[m][k]*w[n][k] + bias[n])),
 * one multiplier / rshift for the whole tensor.  Built on the conv path: prepack
 * with tpuhip_fc_prepack, run with tpuhip_conv2d_i8.  x rows have stride x_cs,
 * y rows stride y_cs. */
int tpuhip_fc_prepack(tpuhip_ctx *ctx, int m, int k, int n, int x_cs, int y_cs, int do_relu,
                      const int8_t *filter_nk, const int32_t *bias, int32_t multiplier,
                      int32_t rshift, tpuhip_conv_weights **out);
/* FullyConnectedOpKernel::invoke (core/fullyconnected.cpp:44-91) for weights packed by
 * tpuhip_fc_prepack.  Matrices of at most 256 rows split K.  With K of 1024 or more, one launch:
 * sixteen waves per 32x32 block of outputs take a sixteenth of K each and add their partial sums
 * in LDS.  With a shorter K, K is divided over workgroups, whose 32x32 int32 partial sums meet
 * in a scratch buffer in device memory that the library allocates with the context's first
 * such call (and grows when a larger layer comes); a second launch adds them up and
 * requantises.  Larger matrices take the conv path.  Same result as tpuhip_conv2d_i8 on the
 * same weights. */
int tpuhip_fc_i8(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y);
/* The two-launch split-K FullyConnected, at any K, for callers that cannot allocate (code under HIP graph capture,
 * serving loops, harnesses that forbid hipMalloc): it has no counterpart in the reference.  The
 * partial sums go to a static array in device memory (4 MiB, one per GPU the library runs
 * on, held until the process ends) whose address is looked up when a context is created; the call
 * itself allocates and frees nothing.  Layers that need more than 1024 partial sums of 32x32 outputs
 * (rows/32 x channels/32 x K splits), or that tpuhip_fc_prepack did not pack for the split-K kernel,
 * are refused with TPUHIP_ERR_INVALID.  All calls on one GPU share the array, so calls that overlap
 * there would race: calls on one stream do not overlap; a call from another context while the last
 * user's stream still has work in flight is refused with TPUHIP_ERR_INVALID (a stream query, no
 * wait); two host threads calling at the same moment on two streams remain the caller's to
 * serialise. */
int tpuhip_fc_i8_noalloc(tpuhip_ctx *ctx, const tpuhip_conv_weights *w, const void *x, void *y);

/* The batched and transposed forms of FullyConnectedOpKernel::invoke (core/fullyconnected.cpp:44-91,
 * shapes by parseFullyConnectedParam, TPUOperationSupport.cpp:568-605): batch = batch_high * batch_low
 * matmuls o_b[m][n] = x_b[m][k] * w_b[n][k]^T + bias_b[n].  With input_transpose the input's logical
 * shape is [batch_high, m, batch_low, k], else [batch, m, k]; with output_transpose the result's is
 * [batch_high, m, batch_low, n], else [batch, m, n].  ReLU, then the per-tensor qdm requantisation with
 * (rshift[i], multiplier[i]) where i = (flat logical index of the RESULT) / (m*n), which is how the
 * reference indexes after its output permute.  x and y are channels-last device tensors whose 4-d
 * views (n, c, h, w; missing dims 1) and channel strides are given: the kernel maps logical indices to
 * them, so no transposed copy is made.  The last logical dim of x must be k, of y n.  Only the logical
 * elements of y are written: bytes between its channel count and its channel stride are the caller's to
 * keep zero (a tensor from tpuhip_malloc + tpuhip_memset, or one every earlier kernel wrote, has them so).
 * The sums are exact int32 sums; the reference's are fp32 (mkldnn_ip), which agree while
 * sum |x * w| + |bias| stays below 2^24 per output -- beyond that bound (possible from about 1000 input
 * channels on) the reference's rounding depends on its summation order and parity is not pinned. */
typedef struct tpuhip_fc_batched_desc {
  int batch_high, batch_low, m, k, n;
  int input_transpose, output_transpose, do_relu;
  int x_c, x_h, x_w, x_cs; /* 4-d view of the input (its n follows from the size) */
  int y_c, y_h, y_w, y_cs; /* 4-d view of the result */
} tpuhip_fc_batched_desc;
typedef struct tpuhip_fc_batched_weights tpuhip_fc_batched_weights;
/* filter: [batch][n][k]; bias: [batch][n] or NULL; multiplier, rshift: [batch] */
int tpuhip_fc_batched_prepack(tpuhip_ctx *ctx, const tpuhip_fc_batched_desc *desc, const int8_t *filter,
                              const int32_t *bias, const int32_t *multiplier, const int32_t *rshift,
                              tpuhip_fc_batched_weights **out);
int tpuhip_fc_batched_destroy(tpuhip_ctx *ctx, tpuhip_fc_batched_weights *w);
int tpuhip_fc_batched_i8(tpuhip_ctx *ctx, const tpuhip_fc_batched_weights *w, const void *x, void *y);

/* ---- EltwiseAdd ---------------------------------------------------------- */

/* Replaces EltwiseAddOpKernel::i8_invoke (core/eltwise.cpp:52-85):
 * y = sat8(floor(relu?(sum_i x_i * multiplier_i) / 2^rshift + 0.5)).
 * All tensors share pixels x cs bytes. nin <= 8. */
int tpuhip_eltwise_add_i8(tpuhip_ctx *ctx, const void *const *xs, int nin,
                          const int8_t *multiplier, int rshift, int do_relu, void *y,
                          size_t bytes);

/* ---- two-input elementwise ops with broadcasting ------------------------------
 * Replaces the INT8 branches of EltwiseMaxOpKernel / EltwiseMinOpKernel / EltwiseMulOpKernel
 * (core/eltwise.cpp:143-189, 233-279, 324-347) and BroadcastAddOpKernel / BroadcastMulOpKernel /
 * BroadcastSubOpKernel (core/broadcast.cpp:45-154).  Every dimension of an operand equals the
 * output's or is 1.  add / sub / max / min: sat8(floor(relu?(op(x0*m0, x1*m1)) / 2^rshift + 0.5));
 * mul: qdm(relu?(x0*x1), rshift, multiplier).  m0, m1 are the int8-converted multipliers,
 * multiplier the uint32-converted one (as int32), rshift the uint32-converted shift. */
enum { TPUHIP_BIN_ADD = 0, TPUHIP_BIN_SUB = 1, TPUHIP_BIN_MAX = 2, TPUHIP_BIN_MIN = 3, TPUHIP_BIN_MUL = 4 };
typedef struct tpuhip_binary_desc {
  int op;
  int n, c, h, w;       /* output */
  int n0, c0, h0, w0;   /* operand 0 */
  int n1, c1, h1, w1;   /* operand 1 */
  int m0, m1;
  int32_t multiplier;
  int rshift;
  int do_relu;
  int x0_cs, x1_cs, y_cs;
} tpuhip_binary_desc;
int tpuhip_binary_i8(tpuhip_ctx *ctx, const tpuhip_binary_desc *d, const void *x0, const void *x1,
                     void *y);

/* ---- Pooling -------------------------------------------------------------- */

/* Field meaning follows parsePoolParam (TPUOperationSupport.cpp:479-522). */
typedef struct tpuhip_pool_desc {
  int n, c, ih, iw, oh, ow, kh, kw, sh, sw, pt, pb, pl, pr;
  int x_cs, y_cs;
} tpuhip_pool_desc;

/* Replaces PoolingOpKernel::invoke, INT8 max (core/pooling.cpp:155-157). */
int tpuhip_pool_max_i8(tpuhip_ctx *ctx, const tpuhip_pool_desc *d, const void *x, void *y);
/* Replaces PoolingOpKernel::invoke, INT8 average, normal path (core/pooling.cpp:147-154):
 * window sum with zero padding, then sat8(floor(sum * multiplier / 2^rshift + 0.5))
 * evaluated in float32 like the reference. */
int tpuhip_pool_avg_i8(tpuhip_ctx *ctx, const tpuhip_pool_desc *d, const void *x, void *y,
                       uint32_t multiplier, uint32_t rshift);

/* ---- 256-entry table ops ---------------------------------------------------- */

/* Replaces the INT8 branch of the LUT activations: y = table[(unsigned char)x]
 * (core/activation.cpp:47-53 and siblings).  table256: 256 int8 on the host.
 * Pad channels (c..cs-1) stay zero. */
int tpuhip_lut_i8(tpuhip_ctx *ctx, const void *x, void *y, const int8_t *table256, size_t pixels,
                  int c, int cs);
/* Replaces LeakyReluOpKernel::invoke, INT8 branch (core/activation.cpp:126-153):
 * builds the 256-entry table from the four scalars and runs tpuhip_lut_i8. */
int tpuhip_leaky_relu_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t pixels, int c, int cs,
                         uint32_t rshift_pos, uint32_t multiplier_pos, uint32_t rshift_neg,
                         uint32_t multiplier_neg);
/* host helper: the table tpuhip_leaky_relu_i8 uses */
int tpuhip_leaky_relu_table(uint32_t rshift_pos, uint32_t multiplier_pos, uint32_t rshift_neg,
                            uint32_t multiplier_neg, int8_t *table256);
/* Replaces ClipOpKernel::invoke, INT8 (core/clip.cpp:29-40); min/max as float. */
int tpuhip_clip_table(float min, float max, uint32_t rshift, uint32_t multiplier,
                      int8_t *table256);
/* Replaces ReluOpKernel::invoke (core/activation.cpp:155-164). */
int tpuhip_relu_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t bytes);

/* INT8 LRN across channels; replaces lrn_int8 / LrnOpKernel::invoke (core/lrn.cpp:104-166, :212-215).
 * sqr_lut256 / power_lut256: the two 256-entry tables quantizeInt8LrnOps writes (values 0..255, the
 * first indexed by the input byte); sum_rshift, lrn_rshift, quant0, quant1: the op's attributes
 * sum_rshift, lrn_rshift, quant_data0, quant_data1.  Refused where the reference's float arithmetic
 * would stop being exact (255 * quant0 * local_size or 255 * 128 * quant1 reaching 2^24). */
int tpuhip_lrn_i8(tpuhip_ctx *ctx, const void *x, void *y, size_t pixels, int c, int cs, int local_size,
                  const uint8_t *sqr_lut256, const uint8_t *power_lut256, int sum_rshift, int lrn_rshift,
                  int quant0, int quant1);
/* One table per channel: y[.., c] = tables[c * 256 + (uint8_t)x[.., c]]; tables is DEVICE memory
 * (c * 256 bytes).  With tpuhip_prelu_tables (host) it replaces PReluOpKernel::invoke, INT8 branch
 * (core/activation.cpp:185-224): slope holds the c float-stored int8 slopes. */
int tpuhip_lut_per_channel_i8(tpuhip_ctx *ctx, const void *x, void *y, const void *tables,
                              size_t pixels, int c, int cs);
int tpuhip_prelu_tables(const float *slope, int c, uint32_t rshift_pos, uint32_t multiplier_pos,
                        uint32_t rshift_neg, int8_t *tables /* c * 256 */);

/* ---- Upsample, Concat ----------------------------------------------------- */

/* Replaces UpsampleOpKernel::invoke (core/upsample.cpp:20-41), nearest. */
int tpuhip_upsample_nearest_i8(tpuhip_ctx *ctx, const void *x, void *y, int n, int c, int ih,
                               int iw, int scale_h, int scale_w, int x_cs, int y_cs);

/* Replaces ConcatOpKernel::invoke (core/concat.cpp:34-90).  axis is the NCHW
 * axis (0..3).  in_dims: nin x 4 ints (n, c, h, w per input); in_cs: channel
 * stride per input.  rshift / multiplier may be NULL (no requant); an input
 * with multiplier 1 and rshift 0 is copied unchanged. */
int tpuhip_concat_i8(tpuhip_ctx *ctx, const void *const *xs, int nin, const int *in_dims,
                     const int *in_cs, int axis, const uint32_t *rshift,
                     const uint32_t *multiplier, int do_relu, void *y, int y_cs);

/* ---- pure data movement, 4-d shapes -----------------------------------------
 * Replaces PadOpKernel, CropOpKernel, PermuteOpKernel, ReorgOpKernel, TileOpKernel,
 * ReverseOpKernel, ShuffleChannelOpKernel, DepthToSpaceOpKernel, SwapChannelOpKernel,
 * DilateOpKernel, ReflectionPadOpKernel (core/pad.cpp:114-141,
 * crop.cpp:44-92, permute.cpp:8-44, reorg.cpp:20-42, tile.cpp:24-42, reverse.cpp:19-42,
 * shuffle_channel.cpp:21-48, depthtospace.cpp:8-80).  p[]:
 *   PAD_CONST / PAD_EDGE  p[0..3] pads at the beginning of n,c,h,w, p[4..7] at the end (constant
 *                         mode: negative = cut; the padding is 0: the reference never reads
 *                         const_val; edge mode: h and w only)
 *   CROP                  p[0..3] crop_offset, p[4..7] steps
 *   PERMUTE               p[0..3] order (output dimension k is input dimension order[k])
 *   REORG                 p[0] stride
 *   TILE                  p[0] axis, p[1] tiles
 *   REVERSE               p[0] axis
 *   SHUFFLE_CHANNEL       p[0] group
 *   DEPTH_TO_SPACE        p[0] upscale factor, p[1] 1 = "DCR" mode, 0 = CRD
 *   SWAP_CHANNEL          p[0..ic-1] channel_order (output channel k is input channel p[k];
 *                         at most 8 channels; core/swap_channel.cpp:21-34)
 *   DILATE                p[0] ins_w, p[1] ins_h (fill values between columns / rows), p[2]
 *                         fill_constant, an int8 value (DilateOpKernel, core/dilate.cpp:11-59)
 *   REFLECTION_PAD        p[0] / p[1] columns added left / right of w, mirrored about the first /
 *                         last column, each less than w (ReflectionPadOpKernel,
 *                         core/reflectionpad.cpp:21-46) */
enum {
  TPUHIP_MOVE_PAD_CONST = 0, TPUHIP_MOVE_PAD_EDGE = 1, TPUHIP_MOVE_CROP = 2, TPUHIP_MOVE_PERMUTE = 3,
  TPUHIP_MOVE_REORG = 4, TPUHIP_MOVE_TILE = 5, TPUHIP_MOVE_REVERSE = 6,
  TPUHIP_MOVE_SHUFFLE_CHANNEL = 7, TPUHIP_MOVE_DEPTH_TO_SPACE = 8, TPUHIP_MOVE_SWAP_CHANNEL = 9,
  TPUHIP_MOVE_DILATE = 10, TPUHIP_MOVE_REFLECTION_PAD = 11
};
typedef struct tpuhip_move_desc {
  int kind;
  int in, ic, ih, iw;   /* input */
  int on, oc, oh, ow;   /* output */
  int x_cs, y_cs;
  int p[8];
} tpuhip_move_desc;
int tpuhip_move_i8(tpuhip_ctx *ctx, const tpuhip_move_desc *d, const void *x, void *y);
/* PermuteOpKernel::invoke (core/permute.cpp:8-44) on DENSE row-major int8 bytes over the full rank
 * (at most 6): y[..] with dimension d of the result = dimension order[d] of the input.  The module
 * interpreter uses it for shapes that are not 4-d, between two layout conversions; the reference
 * folds such shapes to 4-d first (parsePermuteParam, TPUOperationSupport.cpp:690-737) and fails
 * where that cannot be done. */
int tpuhip_permute_flat_i8(tpuhip_ctx *ctx, const void *x_dense, void *y_dense, int rank, const int64_t *in_shape,
                           const int *order);

/* ---- Reduce over consecutive axes ------------------------------------------
 * Replaces ReduceOpKernel::invoke (core/reduce.cpp:54-117) for INT8 tensors.  kind: 0 mean, 1 sum,
 * 2 max, 3 min, over the logical NCHW axes first_axis..last_axis of the input; the result holds
 * the remaining elements in order, shaped out_nchw (with or without the reduced axes kept as 1).
 * In INT8 a mean is a sum whose 1/count lives in the multiplier.  rshift / multiplier: the op's
 * quant operands; (0, 1) means none, which a sum over more than one element refuses because the
 * reference then leaves a raw sum that is no int8 value. */
int tpuhip_reduce_i8(tpuhip_ctx *ctx, int kind, const void *x, void *y, const int *in_nchw, int x_cs,
                     const int *out_nchw, int y_cs, int first_axis, int last_axis, int rshift,
                     uint32_t multiplier);

/* ---- QuantOp at the graph edges -------------------------------------------
 * Replaces QuantOpKernel::invoke (core/quant.cpp:133-166) for the two conversions an INT8 graph
 * has: fp32 -> int8 right after an input (round(src * scale), half away from zero, clamped,
 * :20-30) and int8 -> fp32 (BF16(src * BF16(scale)), :108-116).  The fp32 side is NCHW. */
int tpuhip_quant_f32_to_i8(tpuhip_ctx *ctx, const void *x_nchw_f32, void *y, int n, int c, int h,
                           int w, int cs, float scale);
int tpuhip_dequant_i8_to_f32(tpuhip_ctx *ctx, const void *x, void *y_nchw_f32, int n, int c, int h,
                             int w, int cs, float scale);

/* ---- module interpreter ------------------------------------------------------ */

/* Flat view of the C++ ModuleInterpreter (include/tpuhip/interpreter.hpp), which
 * mirrors MlirModuleInterpreter (include/tpuc/MlirModuleInterpreter.h:32-83) and
 * what pymlir.module exposes on top of it (bindings/python/pymlir.cpp:289-311).
 * Tensors cross this boundary the way the reference passes them: float32 NCHW
 * arrays holding integers. */
typedef struct tpuhip_module tpuhip_module;

/* One TPU-dialect op: what the reference reads from an mlir::Operation. */
typedef struct {
  const char *type;          /* "tpu.conv_2d", "tpu.eltwise_add", ... */
  const char *name;
  const char *quant;         /* "INT8" | "UINT8" | "BF16" | "NONE" */
  const char *param_type;    /* "RSHIFT_AND_M_I32", "RSHIFT_AND_M_I8", "NONE", ... */
  int ndim;
  const int64_t *shape;      /* result shape */
  int n_operands;
  const char *const *operands; /* value / weight names in operand order, "" for none */
  int n_attrs;
  const char *const *attr_keys;
  const double *attr_values;
} tpuhip_op_desc;

/* MlirModuleInterpreter(batch) */
int tpuhip_module_create(int device, int max_batch, tpuhip_module **out);
int tpuhip_module_destroy(tpuhip_module *m);
/* updateWeightMap: one call per tpu.load_weight (MlirModuleInterpreter.cpp:352-369) */
int tpuhip_module_set_weight(tpuhip_module *m, const char *name, const float *data, size_t count);
/* describe the function body: ops in program order, then the returned values */
int tpuhip_module_clear_ops(tpuhip_module *m);
int tpuhip_module_add_op(tpuhip_module *m, const tpuhip_op_desc *op);
int tpuhip_module_set_returns(tpuhip_module *m, const char *const *names, int n);
/* loadModule(module, target_op): builds / refreshes the kernel list; unchanged
 * kernels are kept (MlirModuleInterpreter.cpp:73-83, 118-350).  target_op may be NULL. */
/* Options read at the next tpuhip_module_load: "fuse_eltwise" (default 1: an EltwiseAdd of a conv
 * result runs in that conv's epilogue), "keep_all_tensors" (default 1: every tensor can be read back
 * after an invoke, as with the reference's get_all_tensor; 0: the result of a conv whose only reader
 * is the add fused into it is never written, and reading it back is an error), "pair_convs"
 * (default 1: two convs over the same input with the same window geometry run as one launch). */
int tpuhip_module_set_option(tpuhip_module *m, const char *key, int value);
int tpuhip_module_load(tpuhip_module *m, const char *target_op);
/* setTensor / getTensor (:407-430) */
int tpuhip_module_set_tensor(tpuhip_module *m, const char *name, const float *data, size_t count,
                             int bidx);
/* set_tensor for callers that hold int8 NCHW data already (no counterpart in the reference, whose
 * tensors are float-stored): a quarter of the bytes cross the bus and no host pass checks or converts
 * them.  Not for fp32 graph inputs (a tpu.input in front of a tpu.quant). */
int tpuhip_module_set_tensor_i8(tpuhip_module *m, const char *name, const int8_t *data, size_t count,
                                int bidx);
int tpuhip_module_get_tensor(tpuhip_module *m, const char *name, float *dst, size_t count,
                             int bidx);
/* same tensor as int8 NCHW, without the float detour */
int tpuhip_module_get_tensor_i8(tpuhip_module *m, const char *name, int8_t *dst, size_t count,
                                int bidx);
/* invoke / invokeTo / fastInvokeAllBatch (:371-405).  Work is queued on the
 * module's stream; tpuhip_module_sync (or any get_tensor) waits for it. */
int tpuhip_module_invoke(tpuhip_module *m, int bidx);
int tpuhip_module_invoke_to(tpuhip_module *m, const char *name, int bidx);
int tpuhip_module_fast_invoke_all_batch(tpuhip_module *m, const char *name, int batch);
int tpuhip_module_sync(tpuhip_module *m);
/* getTensorShape / getDataType / getAllTensorName / outputDetails / input_details */
int tpuhip_module_tensor_shape(tpuhip_module *m, const char *name, int64_t *dims8, int *ndim);
const char *tpuhip_module_tensor_dtype(tpuhip_module *m, const char *name);
int tpuhip_module_num_tensors(tpuhip_module *m);
const char *tpuhip_module_tensor_name(tpuhip_module *m, int i);
int tpuhip_module_num_inputs(tpuhip_module *m);
const char *tpuhip_module_input_name(tpuhip_module *m, int i);
int tpuhip_module_num_outputs(tpuhip_module *m);
const char *tpuhip_module_output_name(tpuhip_module *m, int i);
/* kernels in execution order; algo is the conv variant or "" */
int tpuhip_module_num_kernels(tpuhip_module *m);
const char *tpuhip_module_kernel_name(tpuhip_module *m, int i);
const char *tpuhip_module_kernel_algo(tpuhip_module *m, int i);
/* HIP-event time of every kernel in execution order: ms[i] = mean over iters runs */
int tpuhip_module_time_kernels(tpuhip_module *m, int bidx, int iters, float *ms, int capacity);
tpuhip_ctx *tpuhip_module_ctx(tpuhip_module *m);

/* ---- Modules and tensors in the reference's file formats ------------------- */

/* Replaces py_module::load (bindings/python/pymlir.cpp, load / parseMLIRInput) and the first half
 * of tpuc-interpreter's main (tools/tpuc-interpreter/tpuc-interpreter.cpp): parses a TPU-dialect
 * .mlir file in the generic textual form, reads every tpu.load_weight from the .npz its
 * tpu.weight_file names (MlirModuleInterpreter::updateWeightMap, MlirModuleInterpreter.cpp:352-369)
 * and builds the kernels (loadModule).  The weight file is looked up as written, then beside
 * the .mlir. */
int tpuhip_module_load_mlir(tpuhip_module *m, const char *mlir_path, const char *target_op);
/* py_module::getWeightFilePath / op_info (pymlir.cpp parseMLIRInfo): name, op type, quant mode */
const char *tpuhip_module_weight_file(tpuhip_module *m);
int tpuhip_module_num_ops(tpuhip_module *m);
int tpuhip_module_op_info(tpuhip_module *m, int i, const char **name, const char **type,
                          const char **quant);
/* The whole of tpuc-interpreter's main: `<mlir> --tensor-in <npz> [--tensor-out <npz>]
 * [--dump-all-tensor <npz>]`; NULL, "" or "-" leaves an output file out. */
int tpuhip_module_interpret_files(tpuhip_module *m, const char *mlir_path, const char *tensor_in,
                                  const char *tensor_out, const char *dump_all_tensor);
/* Parses only (no GPU, no weights): one text line per weight, op and return value, for tools
 * and tests.  Writes at most capacity bytes (NUL-terminated); *needed gets the full size. */
int tpuhip_mlir_describe(const char *mlir_path, char *buf, size_t capacity, size_t *needed);

/* TensorFile (include/tpuc/Support/TensorFile.h:83-319): an .npz of arrays keyed by name, held in
 * memory and written back as a whole by keep().  mode 0 = openInputTensorFile (read only, must
 * exist), 1 = openOutputTensorFile (starts empty), 2 = read what exists and allow changes. */
typedef struct tpuhip_npz tpuhip_npz;
int tpuhip_npz_open(const char *filename, int mode, tpuhip_npz **out);
int tpuhip_npz_close(tpuhip_npz *f);
int tpuhip_npz_count(tpuhip_npz *f);
const char *tpuhip_npz_name(tpuhip_npz *f, int i);
/* shape (up to 8 dims), numpy kind character ('f', 'i', 'u', 'b') and bytes per element */
int tpuhip_npz_info(tpuhip_npz *f, const char *name, int64_t *dims8, int *ndim, char *kind,
                    int *word_size);
/* readTensor<float>(name, data, count): float32 of exactly count elements, else an error */
int tpuhip_npz_read_f32(tpuhip_npz *f, const char *name, float *dst, size_t count);
/* addTensor: an error if the name is already used */
int tpuhip_npz_add_f32(tpuhip_npz *f, const char *name, const float *data, const int64_t *dims,
                       int ndim);
int tpuhip_npz_delete(tpuhip_npz *f, const char *name);
int tpuhip_npz_keep(tpuhip_npz *f);

/* ---- INT8 quantisation arithmetic (host only, no GPU) ---------------------- */

/* Replace the helpers the reference's --tpu-quant pass uses to turn fp32 weights and two
 * calibration thresholds into the float-stored integer operands of the INT8 kernels
 * (lib/Dialect/TPU/Quantization/QuantizationArithmetic.cpp; drivers in QuantizeInt8.cpp).
 * threshold_x / threshold_y: calibration thresholds of the op's input / output. */

/* QuantizeMultiplier (:182-220): multiplier = quantized * 2^(shift - 31), quantized in [2^30, 2^31) or 0 */
int tpuhip_quantize_multiplier(double multiplier, int32_t *quantized, int *shift);
/* findRShiftAndMultiplierFromQScale (:237-289); qdm != 0: the 32-bit form conv and FC use;
 * else the 8-bit form with max_multiplier (127 in the reference's callers) */
int tpuhip_find_rshift_and_multiplier(double qscale, int qdm, uint32_t max_multiplier, int *rshift,
                                      uint32_t *multiplier);
/* quantizeWeightInt8Multiplier (:741-818) as quantizeInt8ConvOps calls it (QuantizeInt8.cpp:56-166):
 * filter oc x isz, bias oc or NULL, filter_threshold oc or NULL; outputs float-stored integers:
 * new_filter (int8), new_bias (int32), rshift and multiplier per output channel */
int tpuhip_quantize_conv_weights(const float *filter, const float *bias, int64_t oc, int64_t isz,
                                 float threshold_y, float threshold_x, const float *filter_threshold,
                                 float *new_filter, float *new_bias, float *rshift, float *multiplier);
/* quantizeWeightInt8ForFC (:630-690): filter batch x n x k, bias batch x n or NULL, one rshift and
 * multiplier per batch */
int tpuhip_quantize_fc_weights(const float *filter, const float *bias, int64_t batch, int64_t n, int64_t k,
                               float threshold_y, float threshold_x, float *new_filter, float *new_bias,
                               float *rshift, float *multiplier);
/* quantizeInt8RescaleNoWeightOps (QuantizeInt8.cpp:669-854): one rshift and one int8 multiplier per
 * input for eltwise add / max / min and average pooling.  coeff: NULL or one factor per input;
 * divisor: kh * kw of an average pool, else 1 */
int tpuhip_quantize_rescale(const float *threshold_x, int n_inputs, float threshold_y, const float *coeff,
                            int divisor, float *rshift, float *multiplier);
/* quantizeInt8LeakyReluOps (QuantizeInt8.cpp:349-429): out4 = rshift_pos, multiplier_pos, rshift_neg,
 * multiplier_neg */
int tpuhip_quantize_leaky_relu(float negative_slope, float threshold_x, float threshold_y, float *out4);
/* quantizeInt8LutOps (QuantizeInt8.cpp:531-621): the 256-entry table, indexed by the two's-complement
 * byte of the input.  kind: 0 sigmoid, 1 tanh, 2 exp, 3 elu, 4 swish, 5 softplus, 6 log, 7 pow, 8 mish;
 * scale / bias: the op attributes of sigmoid, exp, softplus (1, 0 if none); coeff: pow's exponent.
 * Entries the reference leaves as NaN (log of a negative input) are NaN here too. */
int tpuhip_quantize_lut_table(int kind, float threshold_x, float threshold_y, float scale, float bias,
                              float coeff, float *table256);

/* tpuc-opt --import-calibration-table --calibration-table T --tpu-quant in.mlir -o out.mlir
 * (lib/Dialect/TPU/Quantization/ImportCalibrationTable.cpp:250-415, Quantization.cpp:657-787,
 * QuantizeInt8.cpp): reads an fp32 TPU-dialect function and the weight .npz it names, takes the
 * thresholds of the calibration table (`name threshold [min max]` per line), and writes the INT8
 * function (weights quantised, rescaling operands added, tpu.quant ops at the fp32 edges) with a new
 * weight file -- out_weights, or out.mlir's stem + "_weights.npz" when NULL.  What it writes is
 * what tpuhip_module_load_mlir loads.  Host code only, no GPU.  Op kinds: conv_2d, deconv_2d,
 * fully_connected, eltwise add / max / min / mul, broadcast add / sub / mul, pool_avg_2d,
 * pool_max_2d, relu, leaky_relu, prelu, clip, concat, the table activations (sigmoid, tanh, exp, elu,
 * swish, softplus, log, pow, mish), upsample, pad, crop, permute, reorg, pixelshuffle, tile,
 * reverse, shuffle_channel, swap_channel, mul_const, lrn (with its threshold_parts), reshape;
 * anything else is refused by name.  `missing` (may be NULL)
 * receives, one per line, the ops the table had no threshold for (the reference warns and goes
 * on); *needed = its length + 1. */
int tpuhip_quantize_mlir_files(const char *in_mlir, const char *calibration_table, const char *out_mlir,
                               const char *out_weights, char *missing, size_t capacity, size_t *needed);

#ifdef __cplusplus
}
#endif
#endif /* TPUHIP_H */

// C++ op-level API of tpuhip: the classes a caller of the reference's
// interpreter works with -- TensorData, CPUOpKernel and its per-op subclasses,
// and the module interpreter -- with the same names, members, operand order and
// invoke() contract, running on the MI355X through the C ABI in tpuhip.h.
//
// Differences forced by the environment, and only these:
//   * mlir::Operation& is replaced by OpDesc, a plain description of one TPU
//     dialect op (MLIR is not available to build against); everything the
//     reference reads from the operation -- result shape, name, quant mode and
//     param type, operands, attributes -- is a field of OpDesc;
//   * an activation TensorData lives in HBM as int8 channels-last; the float
//     NCHW view the reference exposes is produced on set/get;
//   * failures throw std::runtime_error where the reference aborts.
//
// Reference: include/tpuc/Interpreter/cpukernel.h:15-159,
// include/tpuc/MlirModuleInterpreter.h:32-83.
#pragma once

#include <cstdint>
#include <list>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "tpuhip.h"

namespace tpuhip {

using SyncedDataShape = std::vector<int64_t>;

// One TPU-dialect operation as the interpreter sees it.
struct OpDesc {
  std::string type;                    // "tpu.conv_2d", "tpu.eltwise_add", ...
  std::string name;                    // getOpName(op)
  SyncedDataShape shape;               // result tensor shape
  std::string quant = "INT8";          // getOpQuant(op): "INT8" | "UINT8" | "BF16" | "NONE"
  std::string param_type = "NONE";     // getOpQuantParamType(op)
  std::vector<std::string> operands;   // value names in operand order; "" is a NoneOp
  std::map<std::string, double> attrs; // numeric attributes (param struct fields, do_relu, axis...)

  double attr(const std::string &key, double dflt) const;
  double attr(const std::string &key) const;  // throws if absent
  std::string signature() const;              // text of everything but the name (dirty check)
};

// A weight tensor as tpu.load_weight yields it: float-stored values
// (MlirModuleInterpreter.cpp:353-369).
struct WeightData {
  std::vector<float> data;
  size_t size() const { return data.size(); }
  float at(size_t i) const { return data.at(i); }
};

// An activation tensor: `batch` slots of one int8 channels-last image set in HBM -- or, at
// the graph edges only (an fp32 input before its QuantOp, the result of a dequantising
// QuantOp), of float NCHW data like the reference's tensors.
// Mirrors mlir::TensorData (cpukernel.h:15-78): size(), set_batch_idx(),
// assign(), tensor(bidx).
class TensorData {
public:
  TensorData(tpuhip_ctx *ctx, int32_t batch, const SyncedDataShape &shape, bool f32 = false);
  ~TensorData();
  TensorData(const TensorData &) = delete;
  TensorData &operator=(const TensorData &) = delete;

  size_t size() const { return size_; }          // logical elements of one slot
  void *data() const { return ptr_; }            // device address of the current slot
  void set_batch_idx(int32_t bidx);
  int32_t batch_idx() const { return cur_; }
  // float-stored NCHW host data -> slot bidx (values must be integers in [-128,127])
  void assign(const float *first, size_t num, int32_t bidx);
  // int8 NCHW host data -> slot bidx, for callers that hold bytes already: a quarter of the
  // float form's transfer and no host pass over the elements
  void assign_i8(const int8_t *first, size_t num, int32_t bidx);
  // slot bidx as float-stored NCHW host data
  std::shared_ptr<std::vector<float>> tensor(int32_t bidx) const;
  // slot bidx as int8 NCHW host data (no float detour)
  void read_i8(int8_t *dst, size_t num, int32_t bidx) const;
  // lays the tensor out again with another channel stride (4 for a tensor of at most 4 channels whose
  // only readers take one dword per pixel, else a multiple of 16); the contents are lost
  void set_channel_stride(int new_cs);

  int32_t batch;
  int n = 1, c = 1, h = 1, w = 1;  // 4-d view of the shape (missing dims are 1)
  bool materialized = true;        // false: no kernel writes this tensor (fused away)
  int cs = 16;                     // channel stride in bytes
  bool f32 = false;                // float NCHW instead of int8 channels-last
  bool is_unsigned = false;        // the bytes hold 0..255 (UINT8 tensors: image data in front of a ScaleLut)
  size_t slot_bytes() const { return f32 ? size_ * sizeof(float) : (size_t)n * h * w * cs; }
  tpuhip_ctx *ctx() const { return ctx_; }

private:
  tpuhip_ctx *ctx_;
  size_t size_;
  void *base_ = nullptr;
  // staging for assign(): a pinned host copy and its fp32 image on the device, made on first use
  void *stage_host_ = nullptr, *stage_dev_ = nullptr;
  void *ptr_ = nullptr;
  int32_t cur_ = 0;
};

enum class DataType { INT8, BF16, FP32 };

using SyncedData = std::shared_ptr<TensorData>;
using SyncedWeight = std::shared_ptr<WeightData>;

struct value_map_t : std::map<std::string, SyncedData> {
  tpuhip_ctx *ctx = nullptr;
  std::map<std::string, SyncedDataShape> shapes;  // result shape of every value
};
using weight_map_t = std::map<std::string, SyncedWeight>;

// One operand: an activation, a weight, or none (cpukernel.cpp:50-73).
struct Operand {
  SyncedData act;
  SyncedWeight weight;
  explicit operator bool() const { return act || weight; }
};

class CPUOpKernel {
public:
  CPUOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
              bool hasOpds = true);
  CPUOpKernel() = delete;
  virtual ~CPUOpKernel() {}

  virtual void set_tensor(const std::vector<float> &data);
  virtual void invoke() = 0;

  std::string get_name() { return name; }
  const std::vector<Operand> &operands() const { return opdTensors; }
  SyncedDataShape get_shape() { return shape; }
  std::string get_data_type();
  void set_name(std::string n) { name = std::move(n); }
  void set_shape(SyncedDataShape &s) { shape = s; }
  void set_datatype(std::string type);
  std::string get_op_type() { return op_type; }
  virtual void dump();
  std::vector<float> get_tensor();
  static std::string generateSignature(OpDesc &op);

  SyncedDataShape shape;
  std::string name;
  std::string op_type;
  size_t size = 0;
  DataType datatype = DataType::FP32;
  OpDesc *op = nullptr;
  std::string signature;
  bool dirty = true;
  static int32_t max_batch_size;

protected:
  void assignOperandTensors(OpDesc &op, const value_map_t &valueMapping,
                            const weight_map_t &weightMapping);
  void assignResultTensor(OpDesc &op, value_map_t &valueMapping);
  void require_int8(const char *what) const;
  tpuhip_ctx *ctx = nullptr;
  std::vector<Operand> opdTensors;
  SyncedData resTensor;
};

// ---- per-op kernels (same class names as the reference's) -----------------

class InputOpKernel : public CPUOpKernel {  // core/input.cpp
public:
  static constexpr const char *OpName = "CPUInputOp";
  InputOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
                std::vector<std::pair<std::string, size_t>> &input_details);
  void invoke() override {}
  void set_tensor(const std::vector<float> &data) override;
};

class Conv2DOpKernel : public CPUOpKernel {  // core/conv.cpp
public:
  static constexpr const char *OpName = "CPUConv2DOp";
  Conv2DOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
      : Conv2DOpKernel(op, valueMapping, weightMapping, false) {}
  ~Conv2DOpKernel() override;
  void invoke() override;
  const char *algo_name() const;
  tpuhip_conv_desc desc{};
  // Fold an EltwiseAdd of (src, this conv's result) into this kernel's epilogue:
  // invoke() then also writes dst.  Results are unchanged; only the module
  // interpreter arranges this (it also silences the eltwise kernel).
  bool can_fuse_add() const;
  void fuse_add(SyncedData src, SyncedData dst, int m_src, int m_conv, int rshift, bool relu);
  // Fold a 256-entry table op on this conv's result (Lut / LeakyRelu / Clip kernels) into
  // the epilogue, ahead of a fused add: invoke() then also writes dst = table[result].
  bool can_fuse_lut() const;
  void fuse_lut(const int8_t *table, SyncedData dst);
  bool has_fused_lut() const { return lut_dst != nullptr; }
  // Run a max pool over this conv's result in the conv's launch (the stem + pool head of the
  // ImageNet networks): invoke() then also writes dst.  Takes no table and no add.
  bool can_fuse_pool(const tpuhip_pool_desc &pool) const;
  void fuse_pool(const tpuhip_pool_desc &pool, SyncedData dst);
  bool has_fused_pool() const { return pool_dst != nullptr; }
  bool has_fused_add() const { return fused.enable != 0; }
  // false: table[result] is not written (only the sum fused behind it)
  void set_store_lut(bool store);
  SyncedData final_result() const { return lut_dst ? lut_dst : output_data; }
  void clear_fusion();
  // false: the conv result itself is not written, only the fused sum (set by the module
  // interpreter when nothing else reads it and the caller asked for outputs only)
  void set_store_result(bool store);
  SyncedData result() const { return output_data; }
  SyncedData input() const { return input_data; }
  // Two convs that read the same tensor through the same window geometry can run as one launch
  // with their filters stacked along the output channels (the input is read once, one launch
  // less).  pair_with packs that and makes `second` a no-op; results are unchanged.  Only the
  // module interpreter arranges this.
  bool can_pair_with(const Conv2DOpKernel &second) const;
  void pair_with(Conv2DOpKernel &second);
  bool is_paired_first() const { return pair_packed != nullptr; }
  bool is_paired_second() const { return paired_into != nullptr; }
  const Conv2DOpKernel *paired_first() const { return paired_into; }
  // host copies of the integer operands are kept until the interpreter has decided about
  // pairing; release_host_weights drops them
  void release_host_weights();
  // dissolves the pair this kernel belongs to (as first or second), leaving no link behind
  void unpair();
  // A pointwise conv (with the add folded behind it, if any) and the pointwise conv that reads its
  // final result can run as one launch (tpuhip_conv2d_chain_*): the intermediate tensor is written
  // once and not read back.  chain_with packs that and makes `next` a no-op; it answers false, and
  // changes nothing, where the library does not cover the pair.  Results are unchanged.  Only the
  // module interpreter arranges this, after the add / table fusions and before the pairing.
  bool can_chain_with(const Conv2DOpKernel &next) const;
  bool chain_with(Conv2DOpKernel &next);
  bool is_chain_first() const { return chain_packed != nullptr; }
  bool is_chain_second() const { return chained_into != nullptr; }
  // dissolves the chain this kernel belongs to (as first or second)
  void unchain();
  // true: this conv runs on the stem path, which reads a pixel of its (at most 4-channel) input as one
  // dword, so the input may lie at a channel stride of 4 instead of 16
  bool reads_dword_pixels() const;
  // tells the packed conv its input's channel stride; false where it cannot take it
  bool set_input_stride(int cs);

protected:
  // transposed: the attributes describe a DeConv2D; it runs as a stride-1 conv over the
  // zero-inserted input with the filter flipped
  Conv2DOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping, bool transposed);

private:
  tpuhip_conv_weights *packed = nullptr;
  SyncedData input_data, output_data;
  SyncedData add_src, add_dst;
  tpuhip_fused_add fused{};
  bool store_result = true;
  SyncedData lut_dst;
  SyncedData pool_dst;
  tpuhip_pool_desc pool_desc{};
  int8_t lut_table[256];
  bool store_lut = true;
  bool plain = false;                      // an ordinary dense conv (not transposed)
  std::vector<int8_t> host_w;
  std::vector<int32_t> host_b, host_m, host_r;
  tpuhip_conv_weights *pair_packed = nullptr;
  Conv2DOpKernel *pair_second = nullptr;   // runs inside this kernel's launch
  Conv2DOpKernel *paired_into = nullptr;   // this kernel's work is done by that one
  tpuhip_conv_chain *chain_packed = nullptr;
  Conv2DOpKernel *chain_second = nullptr;  // runs inside this kernel's launch, on its final result
  Conv2DOpKernel *chained_into = nullptr;  // this kernel's work is done by that one
  mutable std::string algo_text;           // storage behind algo_name() of a paired kernel
};

// core/deconv.cpp:7-73, same operands and epilogue as Conv2D
class DeConv2DOpKernel : public Conv2DOpKernel {
public:
  static constexpr const char *OpName = "CPUDeConv2DOp";
  DeConv2DOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
      : Conv2DOpKernel(op, valueMapping, weightMapping, true) {}
};

class FullyConnectedOpKernel : public CPUOpKernel {  // core/fullyconnected.cpp
public:
  static constexpr const char *OpName = "CPUFullyConnectedOp";
  FullyConnectedOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  ~FullyConnectedOpKernel() override;
  void invoke() override;
  int m = 0, k = 0, n = 0;
  int batch_high = 1, batch_low = 1, batch = 1;   // parseFullyConnectedParam
  bool ltrans = false, otrans = false;            // input_transpose, output_transpose
  // "fc/<conv tile variant it runs as>" (the variant is timed on first use), or "fc/batched"
  const char *algo_name() const;

private:
  mutable std::string algo_text;
  tpuhip_conv_weights *packed = nullptr;              // [m,k] x [n,k]: the MFMA path
  tpuhip_fc_batched_weights *packed_batched = nullptr;  // every other form
  SyncedData input_data, output_data;
};

class EltwiseAddOpKernel : public CPUOpKernel {  // core/eltwise.cpp:7-100
public:
  static constexpr const char *OpName = "CPUEltwiseAddOp";
  EltwiseAddOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;
  // set by the module interpreter when a producing conv computes this op's result
  bool fused_into_producer = false;
  const std::vector<SyncedData> &inputs() const { return inputs_data; }
  SyncedData result() const { return output_data; }
  const std::vector<int8_t> &multipliers() const { return multiplier; }
  int rshift_value() const { return rshift; }
  bool relu() const { return do_relu; }

private:
  std::vector<SyncedData> inputs_data;
  SyncedData output_data;
  std::vector<int8_t> multiplier;
  int rshift = 0;
  bool do_relu = false;
};

// Two-input elementwise ops.  The Eltwise* classes take same-shape inputs followed by
// [n+0]quant_scale [n+1]zeropoint [n+2]rshift [n+3]multiplier (core/eltwise.cpp:102-126);
// the Broadcast* classes two inputs whose dimensions are the result's or 1, followed by
// [2]scale [3]zeropoint [4]rshift [5]multiplier (core/broadcast.cpp:9-43).
class BinaryOpKernel : public CPUOpKernel {
public:
  void invoke() override;

protected:
  BinaryOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping, int op_code,
                 bool broadcast, const char *what);
  tpuhip_binary_desc desc{};
  SyncedData in0, in1, output_data;
};

#define TPUHIP_BINARY_KERNEL(Class, Name, code, bcast)                                        \
  class Class : public BinaryOpKernel {                                                       \
  public:                                                                                     \
    static constexpr const char *OpName = Name;                                               \
    Class(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)                 \
        : BinaryOpKernel(op, valueMapping, weightMapping, code, bcast, Name) {}               \
  };
TPUHIP_BINARY_KERNEL(EltwiseMaxOpKernel, "CPUEltwiseMaxOp", TPUHIP_BIN_MAX, false)   // eltwise.cpp:102
TPUHIP_BINARY_KERNEL(EltwiseMinOpKernel, "CPUEltwiseMinOp", TPUHIP_BIN_MIN, false)   // eltwise.cpp:192
TPUHIP_BINARY_KERNEL(EltwiseMulOpKernel, "CPUEltwiseMulOp", TPUHIP_BIN_MUL, false)   // eltwise.cpp:282
TPUHIP_BINARY_KERNEL(BroadcastAddOpKernel, "CPUBroadcastAddOp", TPUHIP_BIN_ADD, true)   // broadcast.cpp:45
TPUHIP_BINARY_KERNEL(BroadcastMulOpKernel, "CPUBroadcastMulOp", TPUHIP_BIN_MUL, true)   // broadcast.cpp:90
TPUHIP_BINARY_KERNEL(BroadcastSubOpKernel, "CPUBroadcastSubOp", TPUHIP_BIN_SUB, true)   // broadcast.cpp:117
#undef TPUHIP_BINARY_KERNEL

class PoolingOpKernel : public CPUOpKernel {  // core/pooling.cpp
public:
  static constexpr const char *OpName = "CPUPoolingOp";
  PoolingOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

  // set by the module interpreter when the producing conv computes this op's result
  bool fused_into_producer = false;
  bool is_max() const { return !is_avg; }
  const tpuhip_pool_desc &pool_desc() const { return desc; }
  SyncedData input() const { return input_data; }
  SyncedData result() const { return output_data; }

private:
  tpuhip_pool_desc desc{};
  bool is_avg = false;
  uint32_t rshift = 0, multiplier = 0;
  SyncedData input_data, output_data;
};

// 256-entry table ops.  LeakyRelu (core/activation.cpp:104-153), Clip
// (core/clip.cpp) and the y0_table activations -- Sigmoid, Exp, Mish, Swish,
// Elu, SoftPlus, Pow, TanH, Log -- (core/activation.cpp:47-53 and siblings) all
// reduce to one lookup per int8 element.
class LutOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPULutOp";
  LutOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;
  int8_t table[256];
  // set by the module interpreter when the producing conv applies the table itself
  bool fused_into_producer = false;
  SyncedData input() const { return input_data; }
  SyncedData result() const { return output_data; }

protected:
  SyncedData input_data, output_data;
};

class LeakyReluOpKernel : public LutOpKernel {
public:
  static constexpr const char *OpName = "CPULeakyReluOp";
  LeakyReluOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
};

class ClipOpKernel : public LutOpKernel {
public:
  static constexpr const char *OpName = "CPUClipOp";
  ClipOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
};

// ReduceMean / ReduceSum / ReduceMax / ReduceMin (core/reduce.cpp:7-117), INT8.
// operands: [0]input [1]lut [2]mantissa_lut (unused) [3]rshift [4]multiplier; attribute axes
class ReduceOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPUReduceOp";
  ReduceOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  SyncedData input_data, output_data;
  int kind = 0, first_axis = 0, last_axis = 0, rshift = 0;
  uint32_t multiplier = 1;
};

// INT8 LRN (core/lrn.cpp:168-235).  operands: [0]input [1]sqr_lut [2]power_lut [3]scale (unused)
class LrnOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPULrnOp";
  LrnOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  SyncedData input_data, output_data;
  uint8_t sqr_lut[256], power_lut[256];
  int local_size = 0, sum_rshift = 0, lrn_rshift = 0, quant_data0 = 0, quant_data1 = 0;
};

// INT8 ZeroMask (core/zero_mask.cpp:8-35): 127 where the input is non-zero (positive) or zero
// (not positive), else 0.  A function of one byte, so it runs as a table.
class ZeroMaskOpKernel : public LutOpKernel {
public:
  static constexpr const char *OpName = "CPUZeroMaskOp";
  ZeroMaskOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
};

// INT8 MulConst (core/eltwise.cpp:360-401): F32ToInt8(x * const_val, nearest even), optional
// ReLU; const_val is 1, -1 or 0 after the quantisation pass.  Also a table.
class MulConstOpKernel : public LutOpKernel {
public:
  static constexpr const char *OpName = "CPUMulConstOp";
  MulConstOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
};

// operands: [0]input [1]slope (c values) [2..5]unused [6]rshift_pos [7]multiplier_pos
// [8]rshift_neg (core/activation.cpp:165-183).  Realised as one 256-entry table per channel.
class PReluOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPUPReluOp";
  PReluOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  ~PReluOpKernel() override;
  void invoke() override;

private:
  SyncedData input_data, output_data;
  void *tables = nullptr;   // device, c * 256 bytes
};

// core/scale_lut.cpp:7-31: y[n,c,h,w] = table[c * 256 + x[n,c,h,w]], operands [0]input
// [1]table (1 x c x 16 x 16, built by quantizeInt8ScaleLutOps, QuantizeInt8.cpp:623-657, for
// inputs 0..255).  The input must be a UINT8 tensor: with a negative x the reference's index
// lands in the previous channel's table, or throws for channel 0.
class ScaleLutOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPUScaleLutOp";
  ScaleLutOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  ~ScaleLutOpKernel() override;
  void invoke() override;

private:
  SyncedData input_data, output_data;
  void *tables = nullptr;   // device, c * 256 bytes
};

// core/quant.cpp:118-166.  The result type is the op's quant mode ("INT8" or "NONE"); the
// source type is that of the operand tensor.  attrs: scale.
class QuantOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPUQuantOp";
  QuantOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  SyncedData input_data, output_data;
  float scale = 1.0f;
};

class ReluOpKernel : public CPUOpKernel {  // core/activation.cpp:155-164
public:
  static constexpr const char *OpName = "CPUReluOp";
  ReluOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  SyncedData input_data, output_data;
};

class UpsampleOpKernel : public CPUOpKernel {  // core/upsample.cpp
public:
  static constexpr const char *OpName = "CPUUpsampleOp";
  UpsampleOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  int scale_h = 1, scale_w = 1;
  SyncedData input_data, output_data;
};

class ConcatOpKernel : public CPUOpKernel {  // core/concat.cpp
public:
  static constexpr const char *OpName = "CPUConcatOp";
  ConcatOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  void invoke() override;

private:
  int axis = 1;
  size_t input_number = 0;
  bool do_relu = false, need_quant = false;
  std::vector<uint32_t> rshift, multiplier;
  std::vector<SyncedData> inputs_data;
  SyncedData output_data;
};

// Pure data movement (4-d shapes).  Array attributes arrive as numbered scalars:
// pads0..7 + mode_edge (PadOp: pads, mode == "edge"), crop_offset0..3 + steps0..3 (CropOp),
// order0..3 (PermuteOp), stride (ReorgOp), axis + tiles (TileOp), axis (ReverseOp),
// group (ShuffleChannelOp), upscale_factor + mode_dcr (DepthToSpaceOp, mode == "DCR").
class MoveOpKernel : public CPUOpKernel {
public:
  void invoke() override;

protected:
  // any_rank: the subclass also takes shapes that are not 4-d (and then runs a path of its own)
  MoveOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping, const char *what,
               bool any_rank = false);
  tpuhip_move_desc desc{};
  SyncedData input_data, output_data;
};
#define TPUHIP_MOVE_KERNEL(Class, Name)                                         \
  class Class : public MoveOpKernel {                                           \
  public:                                                                       \
    static constexpr const char *OpName = Name;                                 \
    Class(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);  \
  };
TPUHIP_MOVE_KERNEL(PadOpKernel, "CPUPadOp")                          // core/pad.cpp:114-141
TPUHIP_MOVE_KERNEL(CropOpKernel, "CPUCropOp")                        // core/crop.cpp:34-92
// core/permute.cpp:35-44.  4-d shapes run the tiled kernels on the channels-last tensors; shapes of
// rank 2, 3, 5 and 6 (the reference folds those to 4-d where it can, parsePermuteParam,
// TPUOperationSupport.cpp:690-737) go through their row-major bytes: channels-last -> dense,
// permute of the dense bytes over the full rank, dense -> channels-last.
class PermuteOpKernel : public MoveOpKernel {
public:
  static constexpr const char *OpName = "CPUPermuteOp";
  PermuteOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  ~PermuteOpKernel() override;
  void invoke() override;

private:
  bool flat = false;
  int rank = 4;
  int64_t in_shape[6] = {1, 1, 1, 1, 1, 1};
  int order[6] = {0, 1, 2, 3, 4, 5};
  void *dense_in = nullptr, *dense_out = nullptr;
};
TPUHIP_MOVE_KERNEL(ReorgOpKernel, "CPUReorgOp")                      // core/reorg.cpp:8-42
TPUHIP_MOVE_KERNEL(TileOpKernel, "CPUTileOp")                        // core/tile.cpp:8-42
TPUHIP_MOVE_KERNEL(ReverseOpKernel, "CPUReverseOp")                  // core/reverse.cpp:7-42
TPUHIP_MOVE_KERNEL(ShuffleChannelOpKernel, "CPUShuffleChannelOp")    // core/shuffle_channel.cpp:7-48
TPUHIP_MOVE_KERNEL(DepthToSpaceOpKernel, "CPUPixelShuffleOp")        // core/depthtospace.cpp:60-80
TPUHIP_MOVE_KERNEL(DilateOpKernel, "CPUDilateOp")                    // core/dilate.cpp:34-59
TPUHIP_MOVE_KERNEL(ReflectionPadOpKernel, "CPUReflectionPadOp")      // core/reflectionpad.cpp:7-46
TPUHIP_MOVE_KERNEL(SwapChannelOpKernel, "CPUSwapChannelOp")          // core/swap_channel.cpp:8-35
#undef TPUHIP_MOVE_KERNEL

// tpu.reshape whose source and result are not the same bytes in channels-last
// order (the reference aliases the NCHW buffer: MlirModuleInterpreter.cpp:331-338).
class ReshapeOpKernel : public CPUOpKernel {
public:
  static constexpr const char *OpName = "CPUReshapeOp";
  ReshapeOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping);
  ~ReshapeOpKernel() override;
  void invoke() override;
  static bool is_alias(const SyncedDataShape &from, const SyncedDataShape &to);

private:
  SyncedData input_data, output_data;
  void *scratch = nullptr;
};

// ---- module interpreter -------------------------------------------------------

using activations_map_t = std::map<std::string, SyncedData>;
using kernel_map_t = std::map<std::string, std::shared_ptr<CPUOpKernel>>;
using kernel_list_t = std::list<std::shared_ptr<CPUOpKernel>>;

// Mirrors mlir::MlirModuleInterpreter (include/tpuc/MlirModuleInterpreter.h:32-83,
// lib/Dialect/TPU/Interpreter/MlirModuleInterpreter.cpp:73-457).  A "module" is
// the list of OpDesc in program order plus the names the function returns.
struct ModuleDesc {
  std::vector<OpDesc> ops;
  std::vector<std::string> returns;
};

class ModuleInterpreter {
public:
  explicit ModuleInterpreter(int32_t batch = 1, int device = 0);
  ~ModuleInterpreter();

  void loadModule(ModuleDesc &module, std::string target_op);
  void loadModule(ModuleDesc &module) { loadModule(module, ""); }
  // module.load(filename) of pymlir / the first half of tpuc-interpreter's main: parse the
  // TPU-dialect text, read the weights its tpu.weight_file names, build the kernels
  void loadModuleFile(const std::string &mlir_path, std::string target_op = "");
  const std::string &weightFilePath() const { return weight_file_path_; }
  // name, op type, quant mode of every op of the loaded file (pymlir's op_info)
  struct OpInfo { std::string name, type, quant; };
  const std::vector<OpInfo> &opInfo() const { return op_info_; }
  void fastInvokeAllBatch(std::string name, int32_t batch);
  void invokeTo(std::string name, int32_t bidx);
  void invoke(int32_t bidx) { invokeTo("", bidx); }
  void setTensor(std::string &name, const std::vector<float> &data, int32_t bidx);
  // the same from a plain buffer (what a C caller holds): no intermediate vector
  void setTensor(std::string &name, const float *data, size_t count, int32_t bidx);
  // the same from int8 NCHW data (no counterpart in the reference, whose tensors are float-stored)
  void setTensorI8(const std::string &name, const int8_t *data, size_t count, int32_t bidx);
  std::shared_ptr<std::vector<float>> getTensor(std::string &name, int32_t bidx);
  void getTensorI8(const std::string &name, int8_t *dst, size_t num, int32_t bidx);
  std::vector<int64_t> getTensorShape(std::string &name);
  std::string getDataType(std::string &name);
  // the reference's updateWeightMap reads every tpu.load_weight from the npz
  // (MlirModuleInterpreter.cpp:352-369); here the caller hands the arrays over
  void updateWeightMap(const std::string &name, const float *data, size_t count);
  std::vector<std::string> &outputDetails() { return output_details; }
  void dump(std::string &name);
  std::vector<std::string> getAllTensorName();
  void sync();

  // per-kernel HIP-event timing of one invoke (ms per kernel, in kernel_list_ order)
  std::vector<std::pair<std::string, float>> timeKernels(int32_t bidx, int iters);
  // kernels in execution order
  const kernel_list_t &kernels() const { return kernel_list_; }
  tpuhip_ctx *context() const { return ctx_; }
  // conv + eltwise-add fusion (on by default; TPUHIP_FUSE=0 disables); applies at the next loadModule
  bool fuse_eltwise = true;
  // convs over the same input with the same geometry run as one launch (on by default;
  // TPUHIP_PAIR=0 disables); applies at the next loadModule
  bool pair_convs = true;
  // a pointwise conv (+ folded add) followed by the pointwise conv that reads its result: one launch
  bool chain_convs = true;
  // a graph input of at most 4 channels that only stem convs read lies one dword per pixel (a quarter
  // of the bytes of the 16-byte channel stride; on by default; TPUHIP_PACK_INPUT=0 disables)
  bool pack_inputs = true;
  // true (default): every tensor of the graph can be read back after an invoke, like the
  // reference.  false: the result of a conv whose only reader is the add fused into it is
  // never written (reading it back is an error); applies at the next loadModule
  bool keep_all_tensors = true;

  std::vector<std::pair<std::string, size_t>> input_details;
  std::vector<std::string> output_details;
  weight_map_t weightMapping;
  activations_map_t activationMapping;
  value_map_t valueMapping;

private:
  void updateKernelList(ModuleDesc &module, std::string &target_op);
  bool isKernelDirty(std::shared_ptr<CPUOpKernel> &krnl, OpDesc *op);
  void fuseKernels();
  void chainConvs();
  void pairConvs();
  void packInputs();
  void spreadDirtiness();
  // kernels that run as one launch (a conv with the table op / add folded into it, the two
  // convs of a pair): rebuilt by every loadModule
  std::vector<std::vector<CPUOpKernel *>> launch_groups_;
  tpuhip_ctx *ctx_ = nullptr;
  kernel_map_t kernel_map_;
  kernel_list_t kernel_list_;
  std::string weight_file_path_;
  std::vector<OpInfo> op_info_;
};

// tools/tpuc-interpreter/tpuc-interpreter.cpp main(): `mlir --tensor-in in.npz [--tensor-out
// out.npz] [--dump-all-tensor all.npz]`; "" or "-" leaves a file out.
void interpretFiles(ModuleInterpreter &interp, const std::string &mlir_path, const std::string &tensor_in,
                    const std::string &tensor_out, const std::string &dump_all_tensor);

}  // namespace tpuhip

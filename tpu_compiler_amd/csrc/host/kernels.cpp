// Host side of the op-level C++ API: TensorData, CPUOpKernel and the per-op
// kernel classes.  Each class parses its OpDesc the way the reference's
// constructor parses the mlir::Operation, converts the float-stored parameters
// with the reference's own conversions, and invoke() issues the HIP work
// through the C ABI.
#include "tpuhip/interpreter.hpp"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <sstream>

namespace tpuhip {

namespace {

[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error(msg); }

void ck(int status, const char *what) {
  if (status != 0) fail(std::string(what) + ": " + tpuhip_last_error());
}

// (uint32_t)float as x86-64 gcc compiles the reference's implicit and explicit
// conversions: truncate to a 64-bit integer, keep the low 32 bits.
uint32_t f2u32(float f) { return (uint32_t)(uint64_t)(int64_t)f; }

// (int8_t)float the same way (eltwise.cpp:66)
int8_t f2i8(float f) { return (int8_t)(int32_t)f; }

int32_t f2i32(float f) {
  if (!(f > -2147483904.0f)) return INT32_MIN;
  if (!(f < 2147483648.0f)) return INT32_MIN;  // x86 cvttss2si "integer indefinite"
  return (int32_t)f;
}

int8_t weight_to_i8(float v, const std::string &op, const char *role) {
  if (!(v >= -128.0f && v <= 127.0f) || v != std::nearbyint(v))
    fail(op + ": " + role + " value " + std::to_string(v) +
         " is not an int8; only INT8-quantized weights are supported");
  return (int8_t)v;
}

void view4(const SyncedDataShape &s, int *n, int *c, int *h, int *w) {
  if (s.empty() || s.size() > 6) fail("tensor rank " + std::to_string(s.size()) + " not supported");
  int64_t d[4] = {1, 1, 1, 1};
  if (s.size() == 1) {
    d[1] = s[0];
  } else if (s.size() > 4) {
    // ranks 5 and 6 (between the reshapes around a permute): the leading dims fold into n,
    // which keeps the row-major order of the elements
    const size_t lead = s.size() - 3;
    for (size_t i = 0; i < lead; ++i) d[0] *= s[i];
    for (size_t i = 0; i < 3; ++i) d[1 + i] = s[lead + i];
  } else {
    for (size_t i = 0; i < s.size(); ++i) d[i] = s[i];
  }
  for (int i = 0; i < 4; ++i)
    if (d[i] <= 0 || d[i] > INT32_MAX) fail("bad tensor dimension");
  *n = (int)d[0]; *c = (int)d[1]; *h = (int)d[2]; *w = (int)d[3];
}

}  // namespace

// ---------------------------------------------------------------------------
// OpDesc
// ---------------------------------------------------------------------------
double OpDesc::attr(const std::string &key, double dflt) const {
  auto it = attrs.find(key);
  return it == attrs.end() ? dflt : it->second;
}

double OpDesc::attr(const std::string &key) const {
  auto it = attrs.find(key);
  if (it == attrs.end()) fail(type + " '" + name + "': missing attribute " + key);
  return it->second;
}

std::string OpDesc::signature() const {
  std::ostringstream os;
  os << type << "|" << quant << "|" << param_type << "|";
  for (auto d : shape) os << d << "x";
  os << "|";
  for (auto &o : operands) os << o << ",";
  os << "|";
  for (auto &kv : attrs) os << kv.first << "=" << kv.second << ";";
  return os.str();
}

// ---------------------------------------------------------------------------
// TensorData
// ---------------------------------------------------------------------------
TensorData::TensorData(tpuhip_ctx *ctx, int32_t batch_, const SyncedDataShape &shape, bool f32_)
    : batch(batch_), f32(f32_), ctx_(ctx) {
  if (batch < 1) fail("TensorData: batch < 1");
  view4(shape, &n, &c, &h, &w);
  cs = tpuhip_channel_stride(c);
  size_ = (size_t)n * c * h * w;
  ck(tpuhip_malloc(ctx_, slot_bytes() * (size_t)batch, &base_), "TensorData");
  ptr_ = base_;
}

TensorData::~TensorData() {
  if (stage_dev_) tpuhip_free(ctx_, stage_dev_);
  if (stage_host_) tpuhip_host_free(ctx_, stage_host_);
  if (base_) tpuhip_free(ctx_, base_);
}

void TensorData::set_channel_stride(int new_cs) {
  if (f32 || new_cs == cs) return;
  if (new_cs < c || (new_cs % 16 != 0 && new_cs != 4)) fail("TensorData::set_channel_stride: bad stride");
  if (base_) ck(tpuhip_free(ctx_, base_), "TensorData::set_channel_stride");
  base_ = nullptr;
  cs = new_cs;
  ck(tpuhip_malloc(ctx_, slot_bytes() * (size_t)batch, &base_), "TensorData::set_channel_stride");
  ck(tpuhip_memset(ctx_, base_, 0, slot_bytes() * (size_t)batch), "TensorData::set_channel_stride");
  ptr_ = (char *)base_ + slot_bytes() * (size_t)cur_;
}

void TensorData::set_batch_idx(int32_t bidx) {
  if (bidx < 0 || bidx >= batch) fail("TensorData::set_batch_idx: slot out of range");
  ptr_ = (char *)base_ + slot_bytes() * (size_t)bidx;
  cur_ = bidx;
}

void TensorData::assign(const float *first, size_t num, int32_t bidx) {
  if (num != size_) fail("TensorData::assign: size mismatch");
  if (bidx < 0 || bidx >= batch) fail("TensorData::assign: slot out of range");
  if (f32) {
    ck(tpuhip_upload(ctx_, (char *)base_ + slot_bytes() * (size_t)bidx, first, num * sizeof(float)),
       "TensorData::assign");
    return;
  }
  const float lo = is_unsigned ? 0.0f : -128.0f, hi = is_unsigned ? 255.0f : 127.0f;
  if (!stage_host_) ck(tpuhip_host_malloc(ctx_, num * sizeof(float), &stage_host_), "TensorData::assign");
  if (!stage_dev_) ck(tpuhip_malloc(ctx_, num * sizeof(float), &stage_dev_), "TensorData::assign");
  // One pass: copy into the pinned buffer, check that every element is an integer of the
  // tensor's byte range, and let 128..255 travel as the int8 value with the same byte.  No
  // early exit and no library call in the loop, so it vectorises; adding and subtracting
  // 1.5 * 2^23 rounds a float of magnitude below 2^22 to an integer.
  float *stage = static_cast<float *>(stage_host_);
  const float magic = 12582912.0f, wrap_from = is_unsigned ? 128.0f : 1e9f;
  unsigned bad = 0;
  for (size_t i = 0; i < num; ++i) {
    const float v = first[i];
    const float r = (v + magic) - magic;
    bad |= (unsigned)!(v >= lo && v <= hi) | (unsigned)(r != v);
    stage[i] = v >= wrap_from ? v - 256.0f : v;
  }
  if (bad)
    for (size_t i = 0; i < num; ++i)
      if (!(first[i] >= lo && first[i] <= hi) || first[i] != std::nearbyint(first[i]))
        fail("TensorData::assign: element " + std::to_string(i) + " = " + std::to_string(first[i]) +
             (is_unsigned ? " is not a uint8 value" : " is not an int8 value"));
  ck(tpuhip_upload(ctx_, stage_dev_, stage, num * sizeof(float)), "TensorData::assign");
  ck(tpuhip_nchw_f32_to_nhwc_i8(ctx_, stage_dev_, (char *)base_ + slot_bytes() * (size_t)bidx, n, c, h, w,
                                cs),
     "TensorData::assign");
}

void TensorData::assign_i8(const int8_t *first, size_t num, int32_t bidx) {
  if (num != size_) fail("TensorData::assign_i8: size mismatch");
  if (bidx < 0 || bidx >= batch) fail("TensorData::assign_i8: slot out of range");
  if (f32) fail("TensorData::assign_i8: this tensor holds fp32 data");
  // the staging buffers of assign() serve here too (a quarter of them is used)
  if (!stage_host_) ck(tpuhip_host_malloc(ctx_, num * sizeof(float), &stage_host_), "TensorData::assign_i8");
  if (!stage_dev_) ck(tpuhip_malloc(ctx_, num * sizeof(float), &stage_dev_), "TensorData::assign_i8");
  std::memcpy(stage_host_, first, num);
  ck(tpuhip_upload(ctx_, stage_dev_, stage_host_, num), "TensorData::assign_i8");
  ck(tpuhip_nchw_to_nhwc_i8(ctx_, stage_dev_, (char *)base_ + slot_bytes() * (size_t)bidx, n, c, h, w, cs),
     "TensorData::assign_i8");
}

std::shared_ptr<std::vector<float>> TensorData::tensor(int32_t bidx) const {
  if (!materialized)
    fail("TensorData::tensor: this tensor is fused into its consumer and never written "
         "(load the module with keep_all_tensors to read it)");
  if (bidx < 0 || bidx >= batch) fail("TensorData::tensor: slot out of range");
  auto out = std::make_shared<std::vector<float>>(size_);
  if (f32) {
    ck(tpuhip_download(ctx_, out->data(), (char *)base_ + slot_bytes() * (size_t)bidx,
                       size_ * sizeof(float)),
       "TensorData::tensor");
    return out;
  }
  void *tmp = nullptr;
  ck(tpuhip_malloc(ctx_, size_ * sizeof(float), &tmp), "TensorData::tensor");
  int rc = tpuhip_nhwc_i8_to_nchw_f32(ctx_, (char *)base_ + slot_bytes() * (size_t)bidx, tmp, n, c,
                                      h, w, cs);
  if (!rc) rc = tpuhip_download(ctx_, out->data(), tmp, size_ * sizeof(float));
  tpuhip_free(ctx_, tmp);
  ck(rc, "TensorData::tensor");
  if (is_unsigned)
    for (auto &v : *out)
      if (v < 0.0f) v += 256.0f;
  return out;
}

void TensorData::read_i8(int8_t *dst, size_t num, int32_t bidx) const {
  if (!materialized)
    fail("TensorData::read_i8: this tensor is fused into its consumer and never written "
         "(load the module with keep_all_tensors to read it)");
  if (f32) fail("TensorData::read_i8: this tensor holds fp32 data");
  if (num != size_) fail("TensorData::read_i8: size mismatch");
  if (bidx < 0 || bidx >= batch) fail("TensorData::read_i8: slot out of range");
  void *tmp = nullptr;
  ck(tpuhip_malloc(ctx_, size_, &tmp), "TensorData::read_i8");
  int rc = tpuhip_nhwc_to_nchw_i8(ctx_, (char *)base_ + slot_bytes() * (size_t)bidx, tmp, n, c, h, w,
                                  cs);
  if (!rc) rc = tpuhip_download(ctx_, dst, tmp, size_);
  tpuhip_free(ctx_, tmp);
  ck(rc, "TensorData::read_i8");
}

// ---------------------------------------------------------------------------
// CPUOpKernel (core/cpukernel.cpp:6-80)
// ---------------------------------------------------------------------------
int32_t CPUOpKernel::max_batch_size = 1;

CPUOpKernel::CPUOpKernel(OpDesc &op_, value_map_t &valueMapping, weight_map_t &weightMapping,
                         bool hasOpds) {
  ctx = valueMapping.ctx;
  if (!ctx) fail("CPUOpKernel: the value map carries no context");
  shape = op_.shape;
  name = op_.name;
  op_type = op_.type;
  set_datatype(op_.quant);
  size = 1;
  for (auto d : shape) size *= (size_t)d;
  if (hasOpds) assignOperandTensors(op_, valueMapping, weightMapping);
  assignResultTensor(op_, valueMapping);
  signature = generateSignature(op_);
  op = &op_;
}

void CPUOpKernel::set_tensor(const std::vector<float> &) { fail("NOT support set_tensor"); }

std::string CPUOpKernel::get_data_type() {
  if (datatype == DataType::BF16) return "BF16";
  if (datatype == DataType::INT8) return "INT8";
  return "FP32";
}

void CPUOpKernel::set_datatype(std::string type) {
  if (type == "NONE")
    datatype = DataType::FP32;
  else if (type == "BF16")
    datatype = DataType::BF16;
  else if (type == "INT8" || type == "UINT8")
    datatype = DataType::INT8;
  else
    fail("Not support type " + type);
}

void CPUOpKernel::dump() {
  if (shape.empty()) fail("No shape");
  std::string shape_str;
  for (auto &i : shape) shape_str += std::to_string(i) + " ";
  printf("%s\n\tName: %s\n\tShape: %s\n\tDataType: %s\n", op_type.c_str(), name.c_str(),
         shape_str.c_str(), get_data_type().c_str());
}

std::vector<float> CPUOpKernel::get_tensor() {
  // deep copy of the current slot, like the reference
  auto t = resTensor->tensor(resTensor->batch_idx());
  return *t;
}

std::string CPUOpKernel::generateSignature(OpDesc &op) { return op.signature(); }

void CPUOpKernel::assignOperandTensors(OpDesc &op_, const value_map_t &valueMapping,
                                       const weight_map_t &weightMapping) {
  for (auto &opd : op_.operands) {
    Operand o;
    if (opd.empty()) {
      opdTensors.push_back(o);
      continue;
    }
    auto wit = weightMapping.find(opd);
    if (wit != weightMapping.end()) {
      o.weight = wit->second;
    } else {
      auto it = valueMapping.find(opd);
      if (it == valueMapping.end()) fail(op_.name + ": operand '" + opd + "' not found (value mapping false)");
      o.act = it->second;
    }
    opdTensors.push_back(o);
  }
}

void CPUOpKernel::assignResultTensor(OpDesc &op_, value_map_t &valueMapping) {
  // fp32 results exist only where the reference's graphs have them next to INT8 ops: the
  // network input and the dequantising QuantOp
  const bool f32 = datatype == DataType::FP32;
  if (f32 && op_.type != "tpu.input" && op_.type != "tpu.quant")
    fail(op_.type + " '" + op_.name + "': only the INT8 path is implemented on the GPU");
  resTensor = std::make_shared<TensorData>(ctx, max_batch_size, op_.shape, f32);
  resTensor->is_unsigned = !f32 && op_.quant == "UINT8";
  valueMapping[op_.name] = resTensor;
  valueMapping.shapes[op_.name] = op_.shape;
}

void CPUOpKernel::require_int8(const char *what) const {
  if (datatype != DataType::INT8)
    fail(std::string(what) + " '" + name + "': only the INT8 path is implemented on the GPU");
  for (auto &opd : opdTensors) {
    if (opd.act && opd.act->f32)
      fail(std::string(what) + " '" + name + "': an fp32 operand needs a QuantOp in front");
    if (opd.act && opd.act->is_unsigned)
      fail(std::string(what) + " '" + name + "': a UINT8 operand is only read by ScaleLut");
  }
  if (resTensor && resTensor->is_unsigned)
    fail(std::string(what) + " '" + name + "': UINT8 results exist only for the network input");
}

// ---------------------------------------------------------------------------
// Input (core/input.cpp:7-24)
// ---------------------------------------------------------------------------
InputOpKernel::InputOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
                             std::vector<std::pair<std::string, size_t>> &input_details)
    : CPUOpKernel(op, valueMapping, weightMapping, false) {
  input_details.push_back(std::make_pair(name, resTensor->size()));
}

void InputOpKernel::set_tensor(const std::vector<float> &data) {
  if (data.size() != resTensor->size())
    fail(" Input op: [" + name + "] required memsize :" + std::to_string(resTensor->size()) +
         ", input data size: " + std::to_string(data.size()) + ": size not same!");
  resTensor->assign(data.data(), data.size(), resTensor->batch_idx());
}

// ---------------------------------------------------------------------------
// Conv2D (core/conv.cpp:11-104)
// ---------------------------------------------------------------------------
Conv2DOpKernel::Conv2DOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
                               bool transposed)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Conv2D");
  if (opdTensors.size() != 7) fail("Conv2D '" + name + "': expected 7 operands");
  input_data = opdTensors[0].act;
  output_data = resTensor;
  auto filter = opdTensors[1].weight;
  auto bias = opdTensors[2].weight;
  auto quant_rshift = opdTensors[5].weight;
  auto quant_multiplier = opdTensors[6].weight;
  if (!input_data || !filter) fail("Conv2D '" + name + "': input / filter operand missing");
  if (!quant_rshift || !quant_multiplier)
    fail("Conv2D '" + name + "': INT8 conv needs per-channel rshift and multiplier operands");

  // parseConvParam (TPUOperationSupport.cpp:366-428)
  tpuhip_conv_desc &d = desc;
  d.kh = (int)op.attr("kernel_h");
  d.kw = (int)op.attr("kernel_w");
  d.dh = (int)op.attr("dilation_h", 1);
  d.dw = (int)op.attr("dilation_w", 1);
  d.sh = (int)op.attr("stride_h", 1);
  d.sw = (int)op.attr("stride_w", 1);
  d.pt = (int)op.attr("padding_t", 0);
  d.pb = (int)op.attr("padding_b", 0);
  d.pl = (int)op.attr("padding_l", 0);
  d.pr = (int)op.attr("padding_r", 0);
  d.g = (int)op.attr("group", 1);
  d.with_bias = (int)op.attr("with_bias", bias ? 1 : 0);
  d.do_relu = (int)op.attr("do_relu", 0);
  d.ins_h = (int)op.attr("ins_h", 0);
  d.ins_w = (int)op.attr("ins_w", 0);
  if (d.kw == 0) d.kw = 1;
  if (input_data->n != output_data->n) fail("input N not equal to output N");
  d.n = input_data->n; d.ic = input_data->c; d.ih = input_data->h; d.iw = input_data->w;
  d.oc = output_data->c; d.oh = output_data->h; d.ow = output_data->w;
  d.x_cs = input_data->cs;
  d.y_cs = output_data->cs;
  d.relu_first = 0;
  d.algo = (int)op.attr("algo", 0);
  if (d.g <= 0 || d.ic % d.g || d.oc % d.g) fail("Conv2D '" + name + "': bad group");

  const size_t fsz = (size_t)d.oc * (d.ic / d.g) * d.kh * d.kw;
  if (filter->size() != fsz) fail("Conv2D '" + name + "': filter size mismatch");
  if (quant_rshift->size() < (size_t)d.oc || quant_multiplier->size() < (size_t)d.oc)
    fail("Conv2D '" + name + "': rshift / multiplier need one entry per output channel");
  std::vector<int8_t> w8(fsz);
  for (size_t i = 0; i < fsz; ++i) w8[i] = weight_to_i8(filter->at(i), name, "filter");
  if (transposed) {
    // out(oh) = sum x(ih) * w(kh) over ih*sh + kh*dh - pt == oh (MKLDeconv,
    // NativeCpuImplementation.h:194-280) == a stride-1 conv of the input with sh-1 zeros
    // between its rows, the filter flipped, padded by (kh-1)*dh - pt at the top
    if (d.ins_h || d.ins_w) fail("DeConv2D '" + name + "': inserted zeros are not an attribute of a deconv");
    const int pt = (d.kh - 1) * d.dh - d.pt, pl = (d.kw - 1) * d.dw - d.pl;
    if (pt < 0 || pl < 0) fail("DeConv2D '" + name + "': padding larger than the kernel extent");
    const int ihd = (d.ih - 1) * d.sh + 1, iwd = (d.iw - 1) * d.sw + 1;
    d.ins_h = d.sh - 1;
    d.ins_w = d.sw - 1;
    d.sh = d.sw = 1;
    d.pt = pt;
    d.pl = pl;
    d.pb = std::max(0, d.oh + d.dh * (d.kh - 1) - ihd - pt);
    d.pr = std::max(0, d.ow + d.dw * (d.kw - 1) - iwd - pl);
    const size_t plane = (size_t)d.kh * d.kw;
    for (size_t f = 0; f < fsz; f += plane) std::reverse(w8.begin() + f, w8.begin() + f + plane);
  }
  std::vector<int32_t> b32, m32((size_t)d.oc), r32((size_t)d.oc);
  // without with_bias the epilogue adds a zero tensor (conv.cpp:59-61)
  if (d.with_bias) {
    if (!bias || bias->size() < (size_t)d.oc) fail("Conv2D '" + name + "': bias operand missing");
    b32.resize((size_t)d.oc);
    for (int i = 0; i < d.oc; ++i) b32[i] = f2i32(bias->at(i));   // (int32_t)bias[i], :859-861
  }
  for (int i = 0; i < d.oc; ++i) {
    // float -> uint32_t at the call, uint32_t -> int32_t inside (:863-865, :534)
    m32[i] = (int32_t)f2u32(quant_multiplier->at(i));
    r32[i] = (int32_t)f2u32(quant_rshift->at(i));
  }
  ck(tpuhip_conv2d_prepack(ctx, &d, w8.data(), d.with_bias ? b32.data() : nullptr, m32.data(),
                           r32.data(), &packed),
     ("Conv2D '" + name + "'").c_str());
  plain = !transposed && d.g == 1 && !d.ins_h && !d.ins_w && (d.algo == 0 || d.algo == 2 || d.algo >= 16);
  if (plain) {
    host_w = std::move(w8);
    host_b = std::move(b32);
    host_m = std::move(m32);
    host_r = std::move(r32);
  }
}

Conv2DOpKernel::~Conv2DOpKernel() {
  unchain();
  unpair();
  if (packed) tpuhip_conv2d_weights_destroy(ctx, packed);
}

// Dissolves the pair this kernel is part of, from either side, so that neither partner keeps
// a pointer to the other (a partial reload may destroy one of them and keep the other).
void Conv2DOpKernel::unpair() {
  if (pair_packed) {
    tpuhip_conv2d_weights_destroy(ctx, pair_packed);
    pair_packed = nullptr;
  }
  if (pair_second) {
    pair_second->paired_into = nullptr;
    pair_second = nullptr;
  }
  if (paired_into) {
    Conv2DOpKernel *first = paired_into;
    paired_into = nullptr;
    first->pair_second = nullptr;
    first->unpair();   // drops the packed pair, which would still write this kernel's result
  }
}

// Dissolves the chain this kernel is part of, from either side (a partial reload may destroy one
// partner and keep the other).
void Conv2DOpKernel::unchain() {
  if (chain_packed) {
    tpuhip_conv2d_chain_destroy(ctx, chain_packed);
    chain_packed = nullptr;
  }
  if (chain_second) {
    chain_second->chained_into = nullptr;
    chain_second = nullptr;
  }
  if (chained_into) {
    Conv2DOpKernel *first = chained_into;
    chained_into = nullptr;
    first->chain_second = nullptr;
    first->unchain();
  }
}

bool Conv2DOpKernel::can_chain_with(const Conv2DOpKernel &o) const {
  if (this == &o || !plain || !o.plain || host_w.empty() || o.host_w.empty()) return false;
  if (pair_packed || paired_into || o.pair_packed || o.paired_into) return false;
  if (chain_packed || chained_into || o.chain_packed || o.chained_into) return false;
  if (lut_dst || pool_dst || o.fused.enable || o.lut_dst || o.pool_dst) return false;
  if (desc.algo != 0 || o.desc.algo != 0) return false;   // a kernel variant asked for by name stays what it is
  const SyncedData &mid = fused.enable ? add_dst : output_data;
  if (o.input_data.get() != mid.get()) return false;
  return tpuhip_conv2d_can_chain(&desc, &o.desc) != 0;
}

bool Conv2DOpKernel::chain_with(Conv2DOpKernel &next) {
  if (!can_chain_with(next)) return false;
  const int rc = tpuhip_conv2d_chain_prepack(
      ctx, &desc, &next.desc, host_w.data(), desc.with_bias ? host_b.data() : nullptr, host_m.data(), host_r.data(),
      next.host_w.data(), next.desc.with_bias ? next.host_b.data() : nullptr, next.host_m.data(), next.host_r.data(),
      &chain_packed);
  if (rc == TPUHIP_ERR_UNSUPPORTED) return false;   // e.g. a right shift of 0: stays two launches
  ck(rc, ("Conv2D '" + name + "' -> '" + next.name + "'").c_str());
  chain_second = &next;
  next.chained_into = this;
  return true;
}

bool Conv2DOpKernel::reads_dword_pixels() const {
  return packed && !pair_packed && !paired_into && !chain_packed && !chained_into &&
         std::string(tpuhip_conv2d_algo_name(packed)) == "stem";
}

bool Conv2DOpKernel::set_input_stride(int cs) {
  if (!packed || tpuhip_conv2d_set_input_stride(packed, cs) != TPUHIP_OK) return false;
  desc.x_cs = cs;
  return true;
}

void Conv2DOpKernel::release_host_weights() {
  std::vector<int8_t>().swap(host_w);
  std::vector<int32_t>().swap(host_b);
  std::vector<int32_t>().swap(host_m);
  std::vector<int32_t>().swap(host_r);
}

bool Conv2DOpKernel::can_pair_with(const Conv2DOpKernel &o) const {
  if (this == &o || !plain || !o.plain || host_w.empty() || o.host_w.empty()) return false;
  if (pair_packed || paired_into || o.pair_packed || o.paired_into) return false;
  if (chain_packed || chained_into || o.chain_packed || o.chained_into) return false;
  if (fused.enable || lut_dst || pool_dst || o.fused.enable || o.lut_dst || o.pool_dst) return false;
  if (input_data.get() != o.input_data.get() || desc.oc % 128 != 0) return false;
  const tpuhip_conv_desc &a = desc, &b = o.desc;
  return a.kh == b.kh && a.kw == b.kw && a.sh == b.sh && a.sw == b.sw && a.pt == b.pt && a.pb == b.pb &&
         a.pl == b.pl && a.pr == b.pr && a.dh == b.dh && a.dw == b.dw && a.oh == b.oh && a.ow == b.ow;
}

void Conv2DOpKernel::pair_with(Conv2DOpKernel &second) {
  if (!can_pair_with(second)) fail("Conv2D '" + name + "': cannot run together with '" + second.name + "'");
  // the pair runs on the kernel variant asked for the first conv (0: timed on first use)
  tpuhip_conv_desc da = desc, db = second.desc;
  db.algo = da.algo;
  ck(tpuhip_conv2d_prepack_pair(ctx, &da, &db, host_w.data(),
                                desc.with_bias ? host_b.data() : nullptr, host_m.data(), host_r.data(),
                                second.host_w.data(), second.desc.with_bias ? second.host_b.data() : nullptr,
                                second.host_m.data(), second.host_r.data(), &pair_packed),
     ("Conv2D '" + name + "' + '" + second.name + "'").c_str());
  pair_second = &second;
  second.paired_into = this;
}

void Conv2DOpKernel::invoke() {
  if (paired_into || chained_into) return;   // computed by the launch of the conv it is paired / chained with
  if (chain_packed) {
    ck(tpuhip_conv2d_chain_i8(ctx, chain_packed, input_data->data(), store_result ? output_data->data() : nullptr,
                              fused.enable ? add_src->data() : nullptr, fused.enable ? add_dst->data() : nullptr,
                              fused.enable ? &fused : nullptr, chain_second->output_data->data()),
       name.c_str());
    return;
  }
  if (pair_packed) {
    ck(tpuhip_conv2d_pair_i8(ctx, pair_packed, input_data->data(), output_data->data(),
                             pair_second->output_data->data()),
       name.c_str());
    return;
  }
  if (!fused.enable && !lut_dst && !pool_dst) {
    ck(tpuhip_conv2d_i8(ctx, packed, input_data->data(), output_data->data()), name.c_str());
    return;
  }
  tpuhip_conv_post post{};
  if (pool_dst) {
    post.pool = &pool_desc;
    post.pool_out = pool_dst->data();
  }
  if (lut_dst) {
    post.lut = lut_table;
    post.lut_out = store_lut ? lut_dst->data() : nullptr;
  }
  if (fused.enable) {
    post.add = fused;
    post.add_src = add_src->data();
    post.add_out = add_dst->data();
  }
  ck(tpuhip_conv2d_post_i8(ctx, packed, input_data->data(),
                           store_result ? output_data->data() : nullptr, &post),
     name.c_str());
}

bool Conv2DOpKernel::can_fuse_add() const {
  return !pair_packed && !paired_into && std::string(tpuhip_conv2d_algo_name(packed)).rfind("mfma", 0) == 0;
}

bool Conv2DOpKernel::can_fuse_pool(const tpuhip_pool_desc &pool) const {
  return !pair_packed && !paired_into && !lut_dst && !fused.enable &&
         tpuhip_conv2d_can_fuse_pool(ctx, packed, &pool) != 0;
}

void Conv2DOpKernel::fuse_pool(const tpuhip_pool_desc &pool, SyncedData dst) {
  if (!dst) fail("Conv2D '" + name + "': fused pool without a result tensor");
  pool_desc = pool;
  pool_dst = dst;
}

void Conv2DOpKernel::fuse_add(SyncedData src, SyncedData dst, int m_src, int m_conv, int rshift,
                              bool relu) {
  if (!src || !dst || src->slot_bytes() != output_data->slot_bytes() ||
      dst->slot_bytes() != output_data->slot_bytes() || src->cs != output_data->cs ||
      dst->cs != output_data->cs)
    fail("Conv2D '" + name + "': fused add operands must match the conv result's shape");
  add_src = src;
  add_dst = dst;
  fused.enable = 1;
  fused.m_src = m_src;
  fused.m_conv = m_conv;
  fused.rshift = rshift;
  fused.do_relu = relu ? 1 : 0;
}

bool Conv2DOpKernel::can_fuse_lut() const {
  // the packed conv answers for its kernel variant: a tile variant fixed by the caller, or
  // chosen by timing before a table was asked for, may have no table stage in its epilogue
  return tpuhip_conv2d_can_fuse_table(packed) != 0 && !lut_dst && !fused.enable && !pair_packed && !paired_into;
}

void Conv2DOpKernel::fuse_lut(const int8_t *table, SyncedData dst) {
  if (!dst || dst->slot_bytes() != output_data->slot_bytes() || dst->cs != output_data->cs)
    fail("Conv2D '" + name + "': a fused table's result must match the conv result's shape");
  memcpy(lut_table, table, 256);
  lut_dst = dst;
  store_lut = true;
}

void Conv2DOpKernel::set_store_lut(bool store) {
  if (!lut_dst || (!store && !fused.enable))
    fail("Conv2D '" + name + "': only a table with an add fused behind it may go unwritten");
  store_lut = store;
  lut_dst->materialized = store;
}

void Conv2DOpKernel::set_store_result(bool store) {
  if (!store && !fused.enable && !lut_dst && !pool_dst)
    fail("Conv2D '" + name + "': only a fused conv may drop its own result");
  store_result = store;
  output_data->materialized = store;
}

void Conv2DOpKernel::clear_fusion() {
  unchain();
  unpair();
  store_result = true;
  output_data->materialized = true;
  if (lut_dst) lut_dst->materialized = true;
  lut_dst.reset();
  pool_dst.reset();
  store_lut = true;
  fused = tpuhip_fused_add{};
  add_src.reset();
  add_dst.reset();
}

const char *Conv2DOpKernel::algo_name() const {
  if (paired_into || chained_into) {
    algo_text = "with " + (paired_into ? paired_into : chained_into)->name;
    return algo_text.c_str();
  }
  if (chain_packed) return tpuhip_conv2d_chain_name(chain_packed);
  return tpuhip_conv2d_algo_name(pair_packed ? pair_packed : packed);
}

// ---------------------------------------------------------------------------
// FullyConnected (core/fullyconnected.cpp:7-91)
// ---------------------------------------------------------------------------
FullyConnectedOpKernel::FullyConnectedOpKernel(OpDesc &op, value_map_t &valueMapping,
                                               weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("FullyConnected");
  if (opdTensors.size() != 7) fail("FullyConnected '" + name + "': expected 7 operands");
  ltrans = op.attr("input_transpose", 0) != 0;
  otrans = op.attr("output_transpose", 0) != 0;
  input_data = opdTensors[0].act;
  output_data = resTensor;
  auto filter = opdTensors[1].weight;
  auto bias = opdTensors[2].weight;
  auto rshift_data = opdTensors[5].weight;
  auto multiplier_data = opdTensors[6].weight;
  if (!input_data || !filter || !rshift_data || !multiplier_data)
    fail("FullyConnected '" + name + "': operand missing");
  // parseFullyConnectedParam (TPUOperationSupport.cpp:568-605): k and n are the last dims of the
  // input and the result (the filter is [..., n, k]); the batch split comes from the input's shape
  // under input_transpose, from the result's under output_transpose, else from the filter's
  // leading dims -- here its element count over n*k, since weights carry no shape
  const SyncedDataShape &o_s = op.shape;
  auto it = valueMapping.shapes.find(op.operands[0]);
  if (it == valueMapping.shapes.end()) fail("FullyConnected '" + name + "': input shape unknown");
  const SyncedDataShape &a_s = it->second;
  const size_t o_dim = o_s.size();
  if (o_dim < 2 || a_s.empty()) fail("FullyConnected '" + name + "': result must have rank 2 or more");
  n = (int)o_s.back();
  // a rank-2 result is one [m,k] x [n,k] product whatever the input's rank ([m, c, 1, 1] is common):
  // m = a_s[0] (:595-597 with o_dim == 2), k = what is left
  const bool rank2 = o_dim == 2 && !ltrans && !otrans;
  k = rank2 ? (int)(input_data->size() / (size_t)std::max<int64_t>(1, a_s[0])) : (int)a_s.back();
  auto prod = [](const SyncedDataShape &s, size_t from, size_t to) {
    int64_t p = 1;
    for (size_t i = from; i < to; ++i) p *= s[i];
    return p;
  };
  if (ltrans || otrans) {
    const SyncedDataShape &s = ltrans ? a_s : o_s;
    if (s.size() != o_dim || o_dim < 3) fail("FullyConnected '" + name + "': a transposed form needs rank 3 or more");
    batch_low = (int)s[o_dim - 2];
    m = (int)s[o_dim - 3];
    batch_high = (int)prod(s, 0, o_dim - 3);
  } else {
    if (filter->size() % ((size_t)n * k)) fail("FullyConnected '" + name + "': filter size mismatch");
    batch_low = (int)(filter->size() / ((size_t)n * k));
    batch_high = 1;
    m = rank2 ? (int)a_s[0] : batch_low > 1 ? (int)a_s[a_s.size() - 2] : (int)prod(a_s, 0, a_s.size() - 1);
  }
  batch = batch_low * batch_high;
  if (filter->size() != (size_t)batch * n * k) fail("FullyConnected '" + name + "': filter size mismatch");
  if (input_data->size() != (size_t)batch * m * k) fail("FullyConnected '" + name + "': input size mismatch");
  if (output_data->size() != (size_t)batch * m * n) fail("FullyConnected '" + name + "': result size mismatch");
  if (rshift_data->size() < (size_t)batch || multiplier_data->size() < (size_t)batch)
    fail("FullyConnected '" + name + "': one rshift and one multiplier per batch needed");
  std::vector<int8_t> w8(filter->size());
  for (size_t i = 0; i < w8.size(); ++i) w8[i] = weight_to_i8(filter->at(i), name, "filter");
  std::vector<int32_t> b32;
  if (bias) {
    if (bias->size() < (size_t)batch * n) fail("FullyConnected '" + name + "': bias size mismatch");
    b32.resize((size_t)batch * n);
    for (size_t i = 0; i < b32.size(); ++i) b32[i] = f2i32(bias->at(i));
  }
  // (uint32_t)rshift_data->at(i), (uint32_t)multiplier_data->at(i) per block i of the result (:78-87)
  std::vector<int32_t> rs((size_t)batch), mu((size_t)batch);
  for (int i = 0; i < batch; ++i) {
    rs[i] = (int32_t)f2u32(rshift_data->at(i));
    mu[i] = (int32_t)f2u32(multiplier_data->at(i));
  }
  const std::string who = "FullyConnected '" + name + "'";
  const bool plain = rank2 && batch == 1 && input_data->h * input_data->w == 1 && input_data->n == m;
  if (plain) {
    ck(tpuhip_fc_prepack(ctx, m, k, n, input_data->cs, output_data->cs, (int)op.attr("do_relu", 0),
                         w8.data(), bias ? b32.data() : nullptr, mu[0], rs[0], &packed),
       who.c_str());
  } else {
    tpuhip_fc_batched_desc d{};
    d.batch_high = batch_high; d.batch_low = batch_low; d.m = m; d.k = k; d.n = n;
    d.input_transpose = ltrans; d.output_transpose = otrans; d.do_relu = (int)op.attr("do_relu", 0);
    d.x_c = input_data->c; d.x_h = input_data->h; d.x_w = input_data->w; d.x_cs = input_data->cs;
    d.y_c = output_data->c; d.y_h = output_data->h; d.y_w = output_data->w; d.y_cs = output_data->cs;
    ck(tpuhip_fc_batched_prepack(ctx, &d, w8.data(), bias ? b32.data() : nullptr, mu.data(), rs.data(),
                                 &packed_batched),
       who.c_str());
  }
}

FullyConnectedOpKernel::~FullyConnectedOpKernel() {
  if (packed) tpuhip_conv2d_weights_destroy(ctx, packed);
  if (packed_batched) tpuhip_fc_batched_destroy(ctx, packed_batched);
}

const char *FullyConnectedOpKernel::algo_name() const {
  algo_text = packed ? std::string("fc/") + tpuhip_conv2d_algo_name(packed) : std::string("fc/batched");
  return algo_text.c_str();
}

void FullyConnectedOpKernel::invoke() {
  if (packed) ck(tpuhip_fc_i8(ctx, packed, input_data->data(), output_data->data()), name.c_str());
  else ck(tpuhip_fc_batched_i8(ctx, packed_batched, input_data->data(), output_data->data()), name.c_str());
}

// ---------------------------------------------------------------------------
// EltwiseAdd (core/eltwise.cpp:7-100)
// ---------------------------------------------------------------------------
EltwiseAddOpKernel::EltwiseAddOpKernel(OpDesc &op, value_map_t &valueMapping,
                                       weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("EltwiseAdd");
  if (opdTensors.size() < 5) fail("EltwiseAdd '" + name + "': expected inputs + 4 operands");
  const size_t nInputs = opdTensors.size() - 4;
  if (op.param_type == "NONE")
    fail("EltwiseAdd '" + name + "': the unquantized (fp32) fallback is not implemented");
  do_relu = op.attr("do_relu", 0) != 0;
  auto quant_rshift = opdTensors[nInputs + 2].weight;
  auto quant_multiplier = opdTensors[nInputs + 3].weight;
  if (!quant_rshift || !quant_multiplier) fail("EltwiseAdd '" + name + "': rshift / multiplier missing");
  if (quant_multiplier->size() < nInputs || quant_rshift->size() < 1)
    fail("EltwiseAdd '" + name + "': one multiplier per input and one rshift needed");
  rshift = (int)f2u32(quant_rshift->at(0));                                    // :81-83
  for (size_t i = 0; i < nInputs; ++i) multiplier.push_back(f2i8(quant_multiplier->at(i)));  // :66
  for (size_t i = 0; i < nInputs; ++i) {
    auto t = opdTensors[i].act;
    if (!t) fail("EltwiseAdd '" + name + "': input " + std::to_string(i) + " is not an activation");
    if (t->slot_bytes() != resTensor->slot_bytes() || t->size() != resTensor->size())
      fail("EltwiseAdd '" + name + "': input shapes differ");
    inputs_data.push_back(t);
  }
  output_data = resTensor;
}

void EltwiseAddOpKernel::invoke() {
  if (fused_into_producer) return;   // the producing conv wrote this result already
  std::vector<const void *> ptrs;
  for (auto &t : inputs_data) ptrs.push_back(t->data());
  ck(tpuhip_eltwise_add_i8(ctx, ptrs.data(), (int)ptrs.size(), multiplier.data(), rshift,
                           do_relu ? 1 : 0, output_data->data(), output_data->slot_bytes()),
     name.c_str());
}

// ---------------------------------------------------------------------------
// EltwiseMax / Min / Mul (core/eltwise.cpp:102-347), BroadcastAdd / Mul / Sub
// (core/broadcast.cpp:9-154)
// ---------------------------------------------------------------------------
BinaryOpKernel::BinaryOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
                               int op_code, bool broadcast, const char *what)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8(what);
  const std::string who = std::string(what) + " '" + name + "'";
  if (opdTensors.size() != 6) fail(who + ": expected two inputs + 4 quantization operands");
  if (op.param_type == "NONE") fail(who + ": the unquantized (fp32) fallback is not implemented");
  in0 = opdTensors[0].act;
  in1 = opdTensors[1].act;
  output_data = resTensor;
  if (!in0 || !in1) fail(who + ": both inputs must be activations");
  auto quant_rshift = opdTensors[4].weight;
  auto quant_multiplier = opdTensors[5].weight;
  if (!quant_rshift || !quant_multiplier || quant_rshift->size() < 1 || quant_multiplier->size() < 1)
    fail(who + ": rshift / multiplier missing");
  tpuhip_binary_desc &d = desc;
  d.op = op_code;
  d.do_relu = op.attr("do_relu", 0) != 0;
  d.n = output_data->n; d.c = output_data->c; d.h = output_data->h; d.w = output_data->w;
  d.n0 = in0->n; d.c0 = in0->c; d.h0 = in0->h; d.w0 = in0->w;
  d.n1 = in1->n; d.c1 = in1->c; d.h1 = in1->h; d.w1 = in1->w;
  d.x0_cs = in0->cs; d.x1_cs = in1->cs; d.y_cs = output_data->cs;
  if (!broadcast && (in0->size() != output_data->size() || in1->size() != output_data->size()))
    fail(who + ": input shapes differ from the result's");
  d.rshift = (int)f2u32(quant_rshift->at(0));
  if (op_code == TPUHIP_BIN_MUL) {
    d.multiplier = (int32_t)f2u32(quant_multiplier->at(0));   // eltwise.cpp:341-343, broadcast.cpp:110
  } else {
    if (quant_multiplier->size() < 2) fail(who + ": one multiplier per input needed");
    d.m0 = f2i8(quant_multiplier->at(0));                      // eltwise.cpp:160, broadcast.cpp:53
    d.m1 = f2i8(quant_multiplier->at(1));
  }
}

void BinaryOpKernel::invoke() {
  ck(tpuhip_binary_i8(ctx, &desc, in0->data(), in1->data(), output_data->data()), name.c_str());
}

// ---------------------------------------------------------------------------
// Pad, Crop, Permute, Reorg, Tile, Reverse, ShuffleChannel, DepthToSpace
// ---------------------------------------------------------------------------
MoveOpKernel::MoveOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping,
                           const char *what, bool any_rank)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8(what);
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail(std::string(what) + " '" + name + "': input missing");
  if (!any_rank && (op.operands.empty() || valueMapping.shapes[op.operands[0]].size() != 4 || shape.size() != 4))
    fail(std::string(what) + " '" + name + "': only 4-d shapes are supported");
  tpuhip_move_desc &d = desc;
  d.in = input_data->n; d.ic = input_data->c; d.ih = input_data->h; d.iw = input_data->w;
  d.on = output_data->n; d.oc = output_data->c; d.oh = output_data->h; d.ow = output_data->w;
  d.x_cs = input_data->cs;
  d.y_cs = output_data->cs;
}

void MoveOpKernel::invoke() {
  ck(tpuhip_move_i8(ctx, &desc, input_data->data(), output_data->data()), name.c_str());
}

static void numbered(const OpDesc &op, const char *base, int count, int *out, double dflt, bool required) {
  for (int i = 0; i < count; ++i) {
    const std::string key = base + std::to_string(i);
    out[i] = (int)(required ? op.attr(key) : op.attr(key, dflt));
  }
}

PadOpKernel::PadOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w) : MoveOpKernel(op, v, w, "Pad") {
  desc.kind = op.attr("mode_edge", 0) != 0 ? TPUHIP_MOVE_PAD_EDGE : TPUHIP_MOVE_PAD_CONST;
  numbered(op, "pads", 8, desc.p, 0, true);
}
CropOpKernel::CropOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w) : MoveOpKernel(op, v, w, "Crop") {
  desc.kind = TPUHIP_MOVE_CROP;
  numbered(op, "crop_offset", 4, desc.p, 0, true);
  numbered(op, "steps", 4, desc.p + 4, 1, false);   // steps default to 1 (parseCropParam)
}
PermuteOpKernel::PermuteOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "Permute", true) {
  const SyncedDataShape &is = v.shapes[op.operands.at(0)];
  rank = (int)is.size();
  if (rank == 4 && shape.size() == 4) {
    desc.kind = TPUHIP_MOVE_PERMUTE;
    numbered(op, "order", 4, desc.p, 0, true);
    return;
  }
  if (rank < 1 || rank > 6 || (int)shape.size() != rank)
    fail("Permute '" + name + "': ranks 1 to 6 are supported, input and result of the same rank");
  flat = true;
  int seen = 0;
  for (int d = 0; d < rank; ++d) {
    in_shape[d] = is[d];
    order[d] = (int)op.attr("order" + std::to_string(d));
    if (order[d] < 0 || order[d] >= rank) fail("Permute '" + name + "': order[" + std::to_string(d) + "] out of range");
    seen |= 1 << order[d];
    if (shape[d] != is[order[d]]) fail("Permute '" + name + "': result dimension " + std::to_string(d) + " does not match");
  }
  if (seen != (1 << rank) - 1) fail("Permute '" + name + "': order is not a permutation");
  ck(tpuhip_malloc(ctx, input_data->size(), &dense_in), name.c_str());
  ck(tpuhip_malloc(ctx, input_data->size(), &dense_out), name.c_str());
}

PermuteOpKernel::~PermuteOpKernel() {
  if (dense_in) tpuhip_free(ctx, dense_in);
  if (dense_out) tpuhip_free(ctx, dense_out);
}

void PermuteOpKernel::invoke() {
  if (!flat) {
    MoveOpKernel::invoke();
    return;
  }
  ck(tpuhip_nhwc_to_nchw_i8(ctx, input_data->data(), dense_in, input_data->n, input_data->c, input_data->h,
                            input_data->w, input_data->cs),
     name.c_str());
  ck(tpuhip_permute_flat_i8(ctx, dense_in, dense_out, rank, in_shape, order), name.c_str());
  ck(tpuhip_nchw_to_nhwc_i8(ctx, dense_out, output_data->data(), output_data->n, output_data->c, output_data->h,
                            output_data->w, output_data->cs),
     name.c_str());
}
ReorgOpKernel::ReorgOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w) : MoveOpKernel(op, v, w, "Reorg") {
  desc.kind = TPUHIP_MOVE_REORG;
  desc.p[0] = (int)op.attr("stride");
}
TileOpKernel::TileOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w) : MoveOpKernel(op, v, w, "Tile") {
  desc.kind = TPUHIP_MOVE_TILE;
  desc.p[0] = (int)op.attr("axis");
  desc.p[1] = (int)op.attr("tiles");
}
ReverseOpKernel::ReverseOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "Reverse") {
  desc.kind = TPUHIP_MOVE_REVERSE;
  desc.p[0] = (int)op.attr("axis");
}
ShuffleChannelOpKernel::ShuffleChannelOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "ShuffleChannel") {
  desc.kind = TPUHIP_MOVE_SHUFFLE_CHANNEL;
  desc.p[0] = (int)op.attr("group");
}
SwapChannelOpKernel::SwapChannelOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "SwapChannel") {
  desc.kind = TPUHIP_MOVE_SWAP_CHANNEL;
  if (desc.ic > 8) fail("SwapChannel '" + name + "': at most 8 channels");
  for (int k = 0; k < desc.ic; ++k) {
    desc.p[k] = (int)op.attr("channel_order" + std::to_string(k));
    if (desc.p[k] < 0 || desc.p[k] >= desc.ic)
      fail("SwapChannel '" + name + "': channel_order[" + std::to_string(k) + "] = " + std::to_string(desc.p[k]));
  }
}
DilateOpKernel::DilateOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w) : MoveOpKernel(op, v, w, "Dilate") {
  desc.kind = TPUHIP_MOVE_DILATE;
  desc.p[0] = (int)op.attr("ins0", 0);   // ins = [w, h], both optional (core/dilate.cpp:43-47)
  desc.p[1] = (int)op.attr("ins1", 0);
  desc.p[2] = (int)op.attr("fill_constant", 0);
}
ReflectionPadOpKernel::ReflectionPadOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "ReflectionPad") {
  desc.kind = TPUHIP_MOVE_REFLECTION_PAD;
  desc.p[0] = (int)op.attr("pads0");
  desc.p[1] = (int)op.attr("pads1");
}
DepthToSpaceOpKernel::DepthToSpaceOpKernel(OpDesc &op, value_map_t &v, weight_map_t &w)
    : MoveOpKernel(op, v, w, "DepthToSpace") {
  desc.kind = TPUHIP_MOVE_DEPTH_TO_SPACE;
  desc.p[0] = (int)op.attr("upscale_factor");
  desc.p[1] = op.attr("mode_dcr", 0) != 0 ? 1 : 0;
}

// ---------------------------------------------------------------------------
// Pooling (core/pooling.cpp:33-160)
// ---------------------------------------------------------------------------
PoolingOpKernel::PoolingOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Pooling");
  is_avg = op.type == "tpu.pool_avg_2d";
  if (op.attr("do_relu", 0) != 0) fail("Pooling '" + name + "': do_relu is not allowed");  // :59
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail("Pooling '" + name + "': input missing");
  // parsePoolParam (TPUOperationSupport.cpp:479-522)
  tpuhip_pool_desc &d = desc;
  d.kh = (int)op.attr("kernel_h");
  d.kw = (int)op.attr("kernel_w");
  if (d.kw == 0) d.kw = 1;
  d.sh = (int)op.attr("stride_h", 1);
  d.sw = (int)op.attr("stride_w", 1);
  d.pt = (int)op.attr("padding_t", 0);
  d.pb = (int)op.attr("padding_b", 0);
  d.pl = (int)op.attr("padding_l", 0);
  d.pr = (int)op.attr("padding_r", 0);
  d.n = input_data->n; d.c = input_data->c; d.ih = input_data->h; d.iw = input_data->w;
  d.oh = output_data->h; d.ow = output_data->w;
  d.x_cs = input_data->cs;
  d.y_cs = output_data->cs;
  if (output_data->n != d.n || output_data->c != d.c) fail("Pooling '" + name + "': N/C mismatch");
  if (is_avg) {
    if (opdTensors.size() < 5 || !opdTensors[3].weight || !opdTensors[4].weight)
      fail("Pooling '" + name + "': quant_rshift / quant_multiplier is null!");   // :74-79
    rshift = f2u32(opdTensors[3].weight->at(0));
    multiplier = f2u32(opdTensors[4].weight->at(0));
  }
}

void PoolingOpKernel::invoke() {
  if (fused_into_producer) return;   // the producing conv wrote this result already
  if (is_avg)
    ck(tpuhip_pool_avg_i8(ctx, &desc, input_data->data(), output_data->data(), multiplier, rshift),
       name.c_str());
  else
    ck(tpuhip_pool_max_i8(ctx, &desc, input_data->data(), output_data->data()), name.c_str());
}

// ---------------------------------------------------------------------------
// table ops
// ---------------------------------------------------------------------------
LutOpKernel::LutOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8(op.type.c_str());
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail(op.type + " '" + name + "': input missing");
  if (input_data->size() != output_data->size()) fail(op.type + " '" + name + "': shape mismatch");
  memset(table, 0, sizeof(table));
  if (op.type != "tpu.leaky_relu" && op.type != "tpu.clip" && op.type != "tpu.zero_mask" &&
      op.type != "tpu.mul_const") {
    // y0_table_op = opdTensors[1] (core/activation.cpp:34-37): 256 float-stored int8 entries,
    // indexed by the two's-complement byte of the input
    auto y0 = opdTensors.size() > 1 ? opdTensors[1].weight : nullptr;
    if (!y0 || y0->size() < 256) fail(op.type + " '" + name + "': y0 table operand missing");
    for (int i = 0; i < 256; ++i) table[i] = weight_to_i8(y0->at(i), name, "table");
  }
}

void LutOpKernel::invoke() {
  if (fused_into_producer) return;   // the conv that produces the input applies the table
  ck(tpuhip_lut_i8(ctx, input_data->data(), output_data->data(), table,
                   (size_t)input_data->n * input_data->h * input_data->w, input_data->c,
                   input_data->cs),
     name.c_str());
}

QuantOpKernel::QuantOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail("Quant '" + name + "': input missing");
  if (input_data->size() != output_data->size()) fail("Quant '" + name + "': shape mismatch");
  if (input_data->f32 == output_data->f32)
    fail("Quant '" + name + "': only fp32 -> INT8 and INT8 -> fp32 are implemented");
  scale = (float)op.attr("scale");
}

void QuantOpKernel::invoke() {
  const TensorData &q = input_data->f32 ? *output_data : *input_data;   // the int8 side
  if (input_data->f32)
    ck(tpuhip_quant_f32_to_i8(ctx, input_data->data(), output_data->data(), q.n, q.c, q.h, q.w, q.cs,
                              scale),
       name.c_str());
  else
    ck(tpuhip_dequant_i8_to_f32(ctx, input_data->data(), output_data->data(), q.n, q.c, q.h, q.w,
                                q.cs, scale),
       name.c_str());
}

PReluOpKernel::PReluOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("PRelu");
  if (opdTensors.size() < 9) fail("PRelu '" + name + "': expected 9 operands");
  input_data = opdTensors[0].act;
  output_data = resTensor;
  auto slope = opdTensors[1].weight;
  if (!input_data || !slope) fail("PRelu '" + name + "': input / slope missing");
  if (input_data->size() != output_data->size()) fail("PRelu '" + name + "': shape mismatch");
  if ((int)slope->size() < input_data->c) fail("PRelu '" + name + "': one slope per channel needed");
  for (int i = 6; i <= 8; ++i)
    if (!opdTensors[i].weight) fail("PRelu '" + name + "': rshift / multiplier operand missing");
  std::vector<int8_t> host((size_t)input_data->c * 256);
  // rshift operands cast explicitly, the multiplier converted implicitly (activation.cpp:211-217)
  ck(tpuhip_prelu_tables(slope->data.data(), input_data->c, f2u32(opdTensors[6].weight->at(0)),
                         f2u32(opdTensors[7].weight->at(0)), f2u32(opdTensors[8].weight->at(0)),
                         host.data()),
     name.c_str());
  ck(tpuhip_malloc(ctx, host.size(), &tables), name.c_str());
  ck(tpuhip_upload(ctx, tables, host.data(), host.size()), name.c_str());
}

PReluOpKernel::~PReluOpKernel() {
  if (tables) tpuhip_free(ctx, tables);
}

void PReluOpKernel::invoke() {
  ck(tpuhip_lut_per_channel_i8(ctx, input_data->data(), output_data->data(), tables,
                               (size_t)input_data->n * input_data->h * input_data->w,
                               input_data->c, input_data->cs),
     name.c_str());
}

// ---------------------------------------------------------------------------
// ScaleLut (core/scale_lut.cpp:7-31)
// ---------------------------------------------------------------------------
ScaleLutOpKernel::ScaleLutOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  if (datatype != DataType::INT8 || resTensor->is_unsigned)
    fail("ScaleLut '" + name + "': the result is an INT8 tensor");
  if (opdTensors.size() < 2) fail("ScaleLut '" + name + "': expected 2 operands");
  input_data = opdTensors[0].act;
  output_data = resTensor;
  auto table = opdTensors[1].weight;
  if (!input_data || !table) fail("ScaleLut '" + name + "': input / table missing");
  if (input_data->f32) fail("ScaleLut '" + name + "': an fp32 operand needs a QuantOp in front");
  if (!input_data->is_unsigned)
    fail("ScaleLut '" + name + "': the input must be a UINT8 tensor (a negative value would index "
         "the previous channel's table in the reference)");
  if (input_data->size() != output_data->size() || input_data->c != output_data->c)
    fail("ScaleLut '" + name + "': shape mismatch");
  const size_t need = (size_t)input_data->c * 256;
  if (table->size() < need) fail("ScaleLut '" + name + "': the table needs 256 entries per channel");
  std::vector<int8_t> host(need);
  for (size_t i = 0; i < need; ++i) host[i] = weight_to_i8(table->at(i), name, "table");
  ck(tpuhip_malloc(ctx, host.size(), &tables), name.c_str());
  ck(tpuhip_upload(ctx, tables, host.data(), host.size()), name.c_str());
}

ScaleLutOpKernel::~ScaleLutOpKernel() {
  if (tables) tpuhip_free(ctx, tables);
}

void ScaleLutOpKernel::invoke() {
  ck(tpuhip_lut_per_channel_i8(ctx, input_data->data(), output_data->data(), tables,
                               (size_t)input_data->n * input_data->h * input_data->w,
                               input_data->c, input_data->cs),
     name.c_str());
}

LeakyReluOpKernel::LeakyReluOpKernel(OpDesc &op, value_map_t &valueMapping,
                                     weight_map_t &weightMapping)
    : LutOpKernel(op, valueMapping, weightMapping) {
  if (opdTensors.size() < 9) fail("LeakyRelu '" + name + "': expected 9 operands");
  for (int i = 5; i <= 8; ++i)
    if (!opdTensors[i].weight) fail("LeakyRelu '" + name + "': rshift / multiplier operand missing");
  // rshift cast explicitly, multiplier converted implicitly (activation.cpp:137-146)
  ck(tpuhip_leaky_relu_table(f2u32(opdTensors[5].weight->at(0)), f2u32(opdTensors[6].weight->at(0)),
                             f2u32(opdTensors[7].weight->at(0)), f2u32(opdTensors[8].weight->at(0)),
                             table),
     name.c_str());
}

ClipOpKernel::ClipOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : LutOpKernel(op, valueMapping, weightMapping) {
  if (opdTensors.size() < 5 || !opdTensors[3].weight || !opdTensors[4].weight)
    fail("Clip '" + name + "': rshift / multiplier operand missing");
  ck(tpuhip_clip_table((float)op.attr("min"), (float)op.attr("max"),
                       f2u32(opdTensors[3].weight->at(0)), f2u32(opdTensors[4].weight->at(0)),
                       table),
     name.c_str());
}

ReduceOpKernel::ReduceOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Reduce");
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail("Reduce '" + name + "': input missing");
  kind = op.type == "tpu.reduce_mean" ? 0 : op.type == "tpu.reduce_sum" ? 1 : op.type == "tpu.reduce_max" ? 2 : 3;
  // consecutive axes, as the reference asserts (reduce.cpp:33-37)
  int count = 0;
  while (op.attrs.count("axes" + std::to_string(count))) ++count;
  if (count == 0) fail("Reduce '" + name + "': no axes");
  first_axis = (int)op.attr("axes0");
  last_axis = (int)op.attr("axes" + std::to_string(count - 1));
  for (int i = 1; i < count; ++i)
    if ((int)op.attr("axes" + std::to_string(i)) != first_axis + i) fail("Reduce '" + name + "': axes must be consecutive");
  if (first_axis < 0 || last_axis > 3) fail("Reduce '" + name + "': axes outside a 4-D tensor");
  for (const auto &opd : op.operands)
    if (valueMapping.shapes.count(opd) && valueMapping.shapes[opd].size() > 4)
      fail("Reduce '" + name + "': tensor rank " + std::to_string(valueMapping.shapes[opd].size()) + " not supported");
  // quant_rshift = opdTensors[3], quant_multiplier = opdTensors[4]; absent: 0 and 1 (reduce.cpp:14-20)
  if (opdTensors.size() > 3 && opdTensors[3].weight) rshift = (int)f2u32(opdTensors[3].weight->at(0));
  if (opdTensors.size() > 4 && opdTensors[4].weight) multiplier = f2u32(opdTensors[4].weight->at(0));
}

void ReduceOpKernel::invoke() {
  const int in[4] = {input_data->n, input_data->c, input_data->h, input_data->w};
  const int out[4] = {output_data->n, output_data->c, output_data->h, output_data->w};
  ck(tpuhip_reduce_i8(ctx, kind, input_data->data(), output_data->data(), in, input_data->cs, out,
                      output_data->cs, first_axis, last_axis, rshift, multiplier),
     name.c_str());
}

LrnOpKernel::LrnOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Lrn");
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data || input_data->slot_bytes() != output_data->slot_bytes()) fail("Lrn '" + name + "': shape mismatch");
  if (opdTensors.size() < 3 || !opdTensors[1].weight || !opdTensors[2].weight ||
      opdTensors[1].weight->size() < 256 || opdTensors[2].weight->size() < 256)
    fail("Lrn '" + name + "': the sqr / power table operands are missing");
  for (int i = 0; i < 256; ++i) {
    const float s = opdTensors[1].weight->at(i), p = opdTensors[2].weight->at(i);
    if (!(s >= 0 && s <= 255 && s == std::floor(s) && p >= 0 && p <= 255 && p == std::floor(p)))
      fail("Lrn '" + name + "': table entry " + std::to_string(i) + " is not an integer in [0,255]");
    sqr_lut[i] = (uint8_t)s;
    power_lut[i] = (uint8_t)p;
  }
  local_size = (int)op.attr("local_size");
  sum_rshift = (int)op.attr("sum_rshift");
  lrn_rshift = (int)op.attr("lrn_rshift");
  quant_data0 = (int)op.attr("quant_data0");
  quant_data1 = (int)op.attr("quant_data1");
}

void LrnOpKernel::invoke() {
  ck(tpuhip_lrn_i8(ctx, input_data->data(), output_data->data(),
                   (size_t)input_data->n * input_data->h * input_data->w, input_data->c, input_data->cs,
                   local_size, sqr_lut, power_lut, sum_rshift, lrn_rshift, quant_data0, quant_data1),
     name.c_str());
}

ZeroMaskOpKernel::ZeroMaskOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : LutOpKernel(op, valueMapping, weightMapping) {
  const bool positive = op.attr("positive", 0) != 0;
  for (int i = 0; i < 256; ++i) {
    const bool zero = (int8_t)i == 0;
    table[i] = (int8_t)(zero ? (positive ? 0 : 127) : (positive ? 127 : 0));
  }
}

MulConstOpKernel::MulConstOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : LutOpKernel(op, valueMapping, weightMapping) {
  const float const_val = (float)op.attr("const_val");
  const bool do_relu = op.attr("do_relu", 0) != 0;
  for (int i = 0; i < 256; ++i) {
    // F32ToInt(v, 0) on |v|: nearest, ties to even (QuantizationArithmetic.cpp:917-938), saturated
    const float v = (float)(int8_t)i * const_val;
    float integer;
    const float fraction = std::modf(std::fabs(v), &integer);
    int q = (int)integer;
    if (fraction > 0.5f) q += 1;
    else if (fraction == 0.5f && (q & 1)) q += 1;
    if (v < 0) q = -q;
    q = std::max(-128, std::min(127, q));
    table[i] = (int8_t)(do_relu && q < 0 ? 0 : q);
  }
}

ReluOpKernel::ReluOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Relu");
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data || input_data->slot_bytes() != output_data->slot_bytes())
    fail("Relu '" + name + "': shape mismatch");
}

void ReluOpKernel::invoke() {
  ck(tpuhip_relu_i8(ctx, input_data->data(), output_data->data(), output_data->slot_bytes()),
     name.c_str());
}

// ---------------------------------------------------------------------------
// Upsample (core/upsample.cpp:7-41)
// ---------------------------------------------------------------------------
UpsampleOpKernel::UpsampleOpKernel(OpDesc &op, value_map_t &valueMapping,
                                   weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Upsample");
  scale_h = (int)op.attr("scale_h");
  scale_w = (int)op.attr("scale_w");
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data) fail("Upsample '" + name + "': input missing");
  if (output_data->h != input_data->h * scale_h || output_data->w != input_data->w * scale_w ||
      output_data->c != input_data->c || output_data->n != input_data->n)
    fail("Upsample '" + name + "': result shape does not match the scales");
}

void UpsampleOpKernel::invoke() {
  ck(tpuhip_upsample_nearest_i8(ctx, input_data->data(), output_data->data(), input_data->n,
                                input_data->c, input_data->h, input_data->w, scale_h, scale_w,
                                input_data->cs, output_data->cs),
     name.c_str());
}

// ---------------------------------------------------------------------------
// Concat (core/concat.cpp:8-90)
// ---------------------------------------------------------------------------
ConcatOpKernel::ConcatOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Concat");
  axis = (int)op.attr("axis");
  if (opdTensors.size() < 5) fail("Concat '" + name + "': expected inputs + 4 operands");
  input_number = opdTensors.size() - 4;
  do_relu = op.attr("do_relu", 0) != 0;
  auto quant_rshift = opdTensors[input_number + 2].weight;
  auto quant_multiplier = opdTensors[input_number + 3].weight;
  if (quant_rshift && quant_multiplier) {
    need_quant = true;
    if (quant_rshift->size() < input_number || quant_multiplier->size() < input_number)
      fail("Concat '" + name + "': one rshift / multiplier per input needed");
    for (size_t i = 0; i < input_number; ++i) {
      rshift.push_back(f2u32(quant_rshift->at(i)));
      multiplier.push_back(f2u32(quant_multiplier->at(i)));
    }
  }
  for (size_t i = 0; i < input_number; ++i) {
    if (!opdTensors[i].act) fail("Concat '" + name + "': input " + std::to_string(i) + " missing");
    inputs_data.push_back(opdTensors[i].act);
  }
  output_data = resTensor;
  // shapes of rank 2..4 lie in the 4-d view with trailing dims of 1, so the axis keeps its number;
  // a rank-1 shape lies along the channels
  if (axis < 0 || axis >= (int)op.shape.size()) fail("Concat '" + name + "': axis outside the shape");
  // (shapes of rank 5 and 6 fold their leading dimensions, which would renumber the axis)
  if (op.shape.size() > 4) fail("Concat '" + name + "': tensor rank " + std::to_string(op.shape.size()) + " not supported");
  if (op.shape.size() == 1) axis = 1;
}

void ConcatOpKernel::invoke() {
  std::vector<const void *> ptrs;
  std::vector<int> dims, css;
  for (auto &t : inputs_data) {
    ptrs.push_back(t->data());
    dims.insert(dims.end(), {t->n, t->c, t->h, t->w});
    css.push_back(t->cs);
  }
  ck(tpuhip_concat_i8(ctx, ptrs.data(), (int)ptrs.size(), dims.data(), css.data(), axis,
                      need_quant ? rshift.data() : nullptr, need_quant ? multiplier.data() : nullptr,
                      do_relu ? 1 : 0, output_data->data(), output_data->cs),
     name.c_str());
}

// ---------------------------------------------------------------------------
// Reshape that cannot alias
// ---------------------------------------------------------------------------
bool ReshapeOpKernel::is_alias(const SyncedDataShape &from, const SyncedDataShape &to) {
  int n0, c0, h0, w0, n1, c1, h1, w1;
  view4(from, &n0, &c0, &h0, &w0);
  view4(to, &n1, &c1, &h1, &w1);
  if (n0 == n1 && c0 == c1 && h0 == h1 && w0 == w1) return true;
  // [n, c, 1, 1] <-> [n, c]: same bytes in channels-last order
  return h0 * w0 == 1 && h1 * w1 == 1 && n0 == n1 && c0 == c1;
}

ReshapeOpKernel::ReshapeOpKernel(OpDesc &op, value_map_t &valueMapping, weight_map_t &weightMapping)
    : CPUOpKernel(op, valueMapping, weightMapping) {
  require_int8("Reshape");
  input_data = opdTensors.at(0).act;
  output_data = resTensor;
  if (!input_data || input_data->size() != output_data->size())
    fail("Reshape '" + name + "': element count changes");
  ck(tpuhip_malloc(ctx, input_data->size(), &scratch), name.c_str());
}

ReshapeOpKernel::~ReshapeOpKernel() {
  if (scratch) tpuhip_free(ctx, scratch);
}

void ReshapeOpKernel::invoke() {
  // channels-last -> NCHW bytes (which the reshape leaves untouched) -> channels-last
  ck(tpuhip_nhwc_to_nchw_i8(ctx, input_data->data(), scratch, input_data->n, input_data->c,
                            input_data->h, input_data->w, input_data->cs),
     name.c_str());
  ck(tpuhip_nchw_to_nhwc_i8(ctx, scratch, output_data->data(), output_data->n, output_data->c,
                            output_data->h, output_data->w, output_data->cs),
     name.c_str());
}

}  // namespace tpuhip

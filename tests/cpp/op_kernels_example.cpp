// The C++ op-level API used the way the reference's interpreter uses its kernel classes
// (lib/Dialect/TPU/Interpreter/MlirModuleInterpreter.cpp:165-344: one CPUOpKernel subclass per
// op, constructed from the op and the value / weight maps, run with invoke(), read with
// get_tensor()).  Builds input -> conv 3x3 + ReLU -> conv 1x1 -> eltwise add (conv1, conv2) with
// ReLU -> global average pool, writes every tensor and every operand to an .npz through
// TensorFile, and prints the file name.  The GPU test runs this program and checks the tensors
// in the file against the CPU oracle.
#include <cstdio>
#include <memory>
#include <vector>

#include "tpuhip/interpreter.hpp"
#include "tpuhip/tensor_file.hpp"

using namespace tpuhip;

namespace {

uint32_t lcg_state = 12345;
int lcg(int lo, int hi) {   // small deterministic integers
  lcg_state = lcg_state * 1664525u + 1013904223u;
  return lo + (int)((lcg_state >> 8) % (uint32_t)(hi - lo + 1));
}

std::vector<float> ints(size_t n, int lo, int hi) {
  std::vector<float> v(n);
  for (auto &x : v) x = (float)lcg(lo, hi);
  return v;
}

void add_weight(weight_map_t &weights, TensorFile &file, const std::string &name, const std::vector<float> &v,
                const std::vector<int64_t> &shape) {
  auto w = std::make_shared<WeightData>();
  w->data = v;
  weights[name] = w;
  file.addTensor(name, v.data(), shape);
}

OpDesc conv_desc(const std::string &name, const std::string &input, int n, int oc, int hw, int k, int pad, bool relu) {
  OpDesc d;
  d.type = "tpu.conv_2d";
  d.name = name;
  d.shape = {n, oc, hw, hw};
  d.quant = "INT8";
  d.param_type = "RSHIFT_AND_M_I32";
  // input, filter, bias, quant_scale, quant_zeropoint, quant_rshift, quant_multiplier (core/conv.cpp:20-36)
  d.operands = {input, name + "_filter", name + "_bias", "", "", name + "_rshift", name + "_multiplier"};
  d.attrs = {{"kernel_h", k}, {"kernel_w", k}, {"stride_h", 1}, {"stride_w", 1}, {"dilation_h", 1},
             {"dilation_w", 1}, {"padding_t", pad}, {"padding_b", pad}, {"padding_l", pad}, {"padding_r", pad},
             {"group", 1}, {"with_bias", 1}, {"do_relu", relu ? 1 : 0}};
  return d;
}

}  // namespace

int main(int argc, char **argv) {
  const std::string out_path = argc > 1 ? argv[1] : "op_kernels_example.npz";
  const int n = 2, ic = 24, c = 32, hw = 12;
  try {
    tpuhip_ctx *ctx = nullptr;
    if (tpuhip_ctx_create(0, &ctx) != TPUHIP_OK) throw std::runtime_error(tpuhip_last_error());
    CPUOpKernel::max_batch_size = 1;
    value_map_t values;
    values.ctx = ctx;
    weight_map_t weights;
    auto file = openOutputTensorFile(out_path);

    for (const char *name : {"conv1", "conv2"}) {
      const bool first = std::string(name) == "conv1";
      const int cin = first ? ic : c, k = first ? 3 : 1;
      add_weight(weights, *file, std::string(name) + "_filter", ints((size_t)c * cin * k * k, -40, 40), {c, cin, k, k});
      add_weight(weights, *file, std::string(name) + "_bias", ints(c, -3000, 3000), {c});
      add_weight(weights, *file, std::string(name) + "_rshift", ints(c, 7, 11), {c});
      std::vector<float> mult(c);
      for (auto &m : mult) m = (float)(((1 << 23) + lcg(0, (1 << 23) - 1)) * 128ll);   // float32-exact, in [2^30, 2^31)
      add_weight(weights, *file, std::string(name) + "_multiplier", mult, {c});
    }
    add_weight(weights, *file, "add_rshift", {5.0f}, {1});
    add_weight(weights, *file, "add_multiplier", {23.0f, 19.0f}, {2});
    add_weight(weights, *file, "gap_rshift", {13.0f}, {1});
    add_weight(weights, *file, "gap_multiplier", {90.0f}, {1});

    // the ops, in program order, as the dispatch chain of updateKernelList builds them
    std::vector<std::pair<std::string, size_t>> input_details;
    OpDesc d_in;
    d_in.type = "tpu.input";
    d_in.name = "data";
    d_in.shape = {n, ic, hw, hw};
    OpDesc d_c1 = conv_desc("conv1", "data", n, c, hw, 3, 1, true);
    OpDesc d_c2 = conv_desc("conv2", "conv1", n, c, hw, 1, 0, false);
    OpDesc d_add;
    d_add.type = "tpu.eltwise_add";
    d_add.name = "add";
    d_add.shape = {n, c, hw, hw};
    d_add.param_type = "RSHIFT_AND_M_I8";
    d_add.operands = {"conv1", "conv2", "", "", "add_rshift", "add_multiplier"};   // core/eltwise.cpp:12-23
    d_add.attrs = {{"do_relu", 1}};
    OpDesc d_gap;
    d_gap.type = "tpu.pool_avg_2d";
    d_gap.name = "gap";
    d_gap.shape = {n, c, 1, 1};
    d_gap.param_type = "RSHIFT_AND_M_I8";
    d_gap.operands = {"add", "", "", "gap_rshift", "gap_multiplier"};               // core/pooling.cpp:72-82
    d_gap.attrs = {{"kernel_h", hw}, {"kernel_w", hw}, {"stride_h", 1}, {"stride_w", 1}, {"padding_t", 0},
                   {"padding_b", 0}, {"padding_l", 0}, {"padding_r", 0}, {"do_relu", 0}};

    std::vector<std::shared_ptr<CPUOpKernel>> kernel_list;
    auto input = std::make_shared<InputOpKernel>(d_in, values, weights, input_details);
    kernel_list.push_back(input);
    kernel_list.push_back(std::make_shared<Conv2DOpKernel>(d_c1, values, weights));
    kernel_list.push_back(std::make_shared<Conv2DOpKernel>(d_c2, values, weights));
    kernel_list.push_back(std::make_shared<EltwiseAddOpKernel>(d_add, values, weights));
    kernel_list.push_back(std::make_shared<PoolingOpKernel>(d_gap, values, weights));

    const std::vector<float> x = ints((size_t)n * ic * hw * hw, -128, 127);
    input->set_tensor(x);
    for (auto &k : kernel_list) k->invoke();       // invokeTo (MlirModuleInterpreter.cpp:371-381)
    if (tpuhip_sync(ctx) != TPUHIP_OK) throw std::runtime_error(tpuhip_last_error());

    for (auto &k : kernel_list) {
      const std::vector<float> t = k->get_tensor();   // deep copy, float-stored NCHW like the reference
      if (t.size() != k->size) throw std::runtime_error("size mismatch for " + k->get_name());
      file->addTensor(k->get_name(), t.data(), k->get_shape());
      std::printf("%-6s %-18s %s %zu values\n", k->get_name().c_str(), k->get_op_type().c_str(),
                  k->get_data_type().c_str(), t.size());
    }
    file->keep();
    kernel_list.clear();
    input.reset();
    values.clear();
    tpuhip_ctx_destroy(ctx);
    std::printf("wrote %s\n", out_path.c_str());
  } catch (const std::exception &e) {
    std::fprintf(stderr, "op_kernels_example: %s\n", e.what());
    return 1;
  }
  return 0;
}

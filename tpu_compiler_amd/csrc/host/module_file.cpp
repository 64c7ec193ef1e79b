// Loading a module from the files the reference's tools exchange: a TPU-dialect .mlir
// (text) whose tpu.weight_file names an .npz of float32 arrays, and the flow of the
// tpuc-interpreter tool around it.
#include <fstream>
#include <sstream>

#include "tpuhip/interpreter.hpp"
#include "tpuhip/mlir_text.hpp"
#include "tpuhip/tensor_file.hpp"

namespace tpuhip {

namespace {

std::string read_text(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good()) throw std::runtime_error("cannot open '" + path + "'");
  std::ostringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

std::string dir_of(const std::string &path) {
  const size_t k = path.find_last_of('/');
  return k == std::string::npos ? std::string() : path.substr(0, k + 1);
}

bool exists(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  return f.good();
}

// the reference's tools compare names by prefix when several inputs are given
// (tools/tpuc-interpreter/tpuc-interpreter.cpp, name_match)
bool name_match(const std::string &a, const std::string &b) {
  if (a.size() == b.size()) return a == b;
  if (a.size() < b.size()) return a == b.substr(0, a.size());
  return a.substr(0, b.size()) == b;
}

}  // namespace

MlirModule readMlirFile(const std::string &mlir_path) {
  return moduleFromMlir(parseMlirText(read_text(mlir_path)));
}

// updateWeightMap + loadModule of the reference (MlirModuleInterpreter.cpp:352-369, :118-163;
// pymlir.cpp py_module::load): every tpu.load_weight is read from the weight file as float32
// of exactly the element count of its result type.
void ModuleInterpreter::loadModuleFile(const std::string &mlir_path, std::string target_op) {
  MlirModule mm = readMlirFile(mlir_path);
  weight_file_path_ = mm.weight_file;
  op_info_.clear();
  for (auto &o : mm.module.ops) op_info_.push_back({o.name, o.type, o.quant});
  if (!mm.weights.empty()) {
    if (mm.weight_file.empty()) throw std::runtime_error(mlir_path + ": tpu.load_weight without a tpu.weight_file");
    // as written (relative to the working directory, like the reference), else beside the .mlir
    std::string wpath = mm.weight_file;
    if (!exists(wpath) && wpath[0] != '/' && exists(dir_of(mlir_path) + wpath)) wpath = dir_of(mlir_path) + wpath;
    TensorFile wfile(wpath, true);
    std::vector<float> data;
    for (auto &w : mm.weights) {
      size_t count = 1;
      for (auto v : w.shape) {
        if (v < 0) throw std::runtime_error("weight '" + w.name + "': dynamic shape");
        count *= (size_t)v;
      }
      data.resize(count);
      if (!wfile.readTensor(w.name, data.data(), count)) {
        auto *a = wfile.find(w.name);
        if (!a) throw std::runtime_error("failed to find tensor " + w.name + " to read in " + wpath);
        // beyond the reference's float-stored files: arrays kept with their integer storage type
        // (int8 filters, int32 biases, ...) are widened to float
        std::vector<float> wide;
        std::vector<int64_t> wshape;
        if (wfile.readTensorAsFloat(w.name, wide, wshape) && wide.size() == count) {
          updateWeightMap(w.name, wide.data(), count);
          continue;
        }
        throw std::runtime_error("size does not match for tensor " + w.name + " in " + wpath + " (float32 x " +
                                 std::to_string(count) + " expected)");
      }
      updateWeightMap(w.name, data.data(), count);
    }
  }
  loadModule(mm.module, target_op);
}

// main() of tools/tpuc-interpreter/tpuc-interpreter.cpp: load, read every array of the input
// npz, bind them to the inputs (one input: whatever its name; several: by name prefix), run,
// write the outputs and / or every tensor.
void interpretFiles(ModuleInterpreter &interp, const std::string &mlir_path, const std::string &tensor_in,
                    const std::string &tensor_out, const std::string &dump_all_tensor) {
  auto inputs = openInputTensorFile(tensor_in);
  std::vector<std::string> names;
  std::vector<std::vector<float>> tensors;
  std::vector<std::vector<int64_t>> shapes;
  inputs->readAllTensors(names, tensors, shapes);

  interp.loadModuleFile(mlir_path);
  auto &details = interp.input_details;
  if (details.size() != tensors.size())
    throw std::runtime_error("Input number not same, needed is " + std::to_string(details.size()) + ", get " +
                             std::to_string(tensors.size()));
  if (tensors.size() == 1) {
    interp.setTensor(details[0].first, tensors[0], 0);
  } else {
    for (size_t i = 0; i < tensors.size(); ++i) {
      size_t j = 0;
      for (; j < details.size(); ++j)
        if (name_match(names[i], details[j].first)) break;
      if (j == details.size()) throw std::runtime_error("not find target tensor in input npz: " + names[i]);
      if (tensors[i].size() != details[j].second)
        throw std::runtime_error("input tensor size not same, needed is " + std::to_string(details[j].second) +
                                 ", get " + std::to_string(tensors[i].size()));
      interp.setTensor(details[j].first, tensors[i], 0);
    }
  }
  interp.invoke(0);
  if (!tensor_out.empty() && tensor_out != "-") {
    auto out = openOutputTensorFile(tensor_out);
    for (auto &name : interp.output_details) {
      std::string n = name;
      auto data = interp.getTensor(n, 0);
      out->addTensor(name, data->data(), interp.getTensorShape(n));
    }
    out->keep();
  }
  if (!dump_all_tensor.empty() && dump_all_tensor != "-") {
    auto out = openOutputTensorFile(dump_all_tensor);
    for (auto &name : interp.getAllTensorName()) {
      std::string n = name;
      auto data = interp.getTensor(n, 0);
      out->addTensor(name, data->data(), interp.getTensorShape(n));
    }
    out->keep();
  }
}

}  // namespace tpuhip

// The producer of the graphs the INT8 interpreter runs: what
//   tpuc-opt --import-calibration-table --calibration-table T --tpu-quant  in.mlir -o out.mlir
// does to an fp32 TPU-dialect function and its weight file
// (lib/Dialect/TPU/Quantization/ImportCalibrationTable.cpp, Quantization.cpp, QuantizeInt8.cpp),
// for the op kinds the INT8 kernels of this library execute.  It works on the parsed text
// (MlirFunc), so attributes it does not know pass through untouched, and it is host code only.
#pragma once

#include <cstdint>
#include <map>
#include <string>
#include <vector>

#include "tpuhip/mlir_text.hpp"

namespace tpuhip {

// The weight tensors a function's tpu.load_weight ops name, in memory.
struct WeightTensor {
  std::vector<int64_t> shape;
  std::vector<float> data;
};
using WeightStore = std::map<std::string, WeightTensor>;

// A calibration table: `name threshold` or `name threshold min max` per line, `#` comments,
// `weight name t0 t1 ...` per-channel filter thresholds, `bitwidth name n` (read and ignored)
// (ImportCalibrationTable.cpp:253-313).  Any other line is an error.
struct CalibrationTable {
  std::map<std::string, float> threshold;
  std::map<std::string, std::vector<float>> weight_threshold;
};
CalibrationTable parseCalibrationTable(const std::string &text);

// ImportCalibrationTablePass::runOnFunction (ImportCalibrationTable.cpp:250-415): writes
// quant.threshold (and param_type "THRESHOLD") of every op that carries a quant attribute,
// 1.0 for sigmoid and tanh whatever the table says, then makes the thresholds on both sides
// of the ops that cannot rescale agree: concat inputs with one use take the concat's
// (:152-178), the producer with one use of a leaky relu / relu / crop / max pool takes the
// op's (:52-93), then the remaining pass-through ops take their producer's (:184-208).
// Returns the names of the ops the table has no entry for (the reference warns and goes on).
std::vector<std::string> importCalibrationTable(MlirFunc &func, const CalibrationTable &table);

// TpuQuantPass::runOnFunction in INT8 mode (Quantization.cpp:657-787): every op but input and
// reshape gets quant.mode "INT8", its weights and rescaling operands are computed by the
// per-op routines of QuantizeInt8.cpp (new tensors are added to `weights`, new
// tpu.load_weight ops to the function), its result becomes si8, and tpu.quant ops are
// inserted where an fp32 value meets an INT8 op and the other way round
// (insertQuantOp, Quantization.cpp:99-255).  Throws std::runtime_error naming the op for a
// kind outside the INT8 interpreter's set, and where a pass-through op has different
// thresholds on its two sides.
void quantizeInt8(MlirFunc &func, WeightStore &weights);

// Reads every tpu.load_weight of `func` from the .npz its tpu.weight_file names (looked up as
// written, else beside mlir_path).
WeightStore readWeights(const MlirFunc &func, const std::string &mlir_path);

// The whole tool: in.mlir (+ its weight file) and a calibration table -> out.mlir and
// out_weights (an .npz holding exactly the tensors out.mlir loads; default: out.mlir's stem +
// "_weights.npz", recorded in the text by base name).  Returns the ops without a table entry.
std::vector<std::string> quantizeFiles(const std::string &in_mlir, const std::string &calibration_table,
                                       const std::string &out_mlir, std::string out_weights = "");

}  // namespace tpuhip

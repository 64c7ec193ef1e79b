// Reader for the textual form of a TPU-dialect module: the generic operation syntax
// `%r = "tpu.op"(%a, %b) {attr = value, ...} : (types) -> type` inside one `func`, which is
// what the reference's tools exchange between passes and what tpuc-interpreter and
// pymlir's module.load() parse with MLIR itself (tools/tpuc-interpreter/tpuc-interpreter.cpp,
// parseMLIRInput; bindings/python/pymlir.cpp, py_module::load).  MLIR is not available to
// build against, so the subset those files use is parsed by hand: SSA ids, string op
// names, attribute dictionaries (integers, floats, booleans, strings, arrays, nested
// dictionaries, anything else skipped by bracket matching), tensor / memref / none types,
// `return`, comments and trailing loc(...).
//
// moduleFromMlir turns the parsed function into the ModuleDesc the interpreter loads:
// what getOpName / getOpQuant / getOpQuantParamType and the param structs give the
// reference's kernels (lib/Dialect/TPU/IR/TPUOperationSupport.cpp) becomes OpDesc fields.
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

#include "tpuhip/interpreter.hpp"

namespace tpuhip {

struct MlirAttr {
  enum Kind { Int, Float, Bool, String, Array, Dict, Unit, Other };
  Kind kind = Unit;
  double num = 0;                 // Int / Float / Bool
  std::string ty;                 // Int / Float: the type written after ':' ("i32", "f32", ...), "" if none
  std::string str;                // String: the unescaped text; Other: the raw text
  std::vector<MlirAttr> items;    // Array
  std::vector<std::pair<std::string, MlirAttr>> fields;   // Dict, in file order
  const MlirAttr *get(const std::string &key) const;      // Dict lookup, nullptr if absent
};

struct MlirType {
  std::string text;               // as written
  bool shaped = false;            // tensor<...> or memref<...>
  std::vector<int64_t> shape;     // -1 for a dynamic dimension
  std::string elem;               // "f32", "si8", "i8", "ui8", "bf16", ...
};

struct MlirOp {
  std::vector<std::string> results;    // SSA ids without '%', "%5:2" gives "5#0", "5#1"
  std::string opname;                  // "tpu.conv_2d", "std.return", ...
  std::vector<std::string> operands;   // SSA ids without '%'
  MlirAttr attrs;                      // Dict (empty when the op has none)
  std::vector<MlirType> operand_types, result_types;
  int line = 0;
};

struct MlirFunc {
  std::string name;
  std::vector<std::pair<std::string, MlirType>> args;   // id without '%', type
  std::vector<MlirType> results;
  MlirAttr attrs;                                       // `attributes {...}` of the func
  std::vector<MlirOp> ops;                              // in program order, the return included
};

// Parses the first func of the text.  Throws std::runtime_error("mlir:<line>: ...").
MlirFunc parseMlirText(const std::string &text);

// The function back as text in the same generic syntax (what parseMlirText reads and what the
// reference's tools read): numbers keep the type they were written with (i32 / f32 when they
// had none), floats print as %e where that reads back to the same float and as their bit
// pattern otherwise, attribute values the reader did not understand are written back verbatim.
std::string printMlir(const MlirFunc &func);
// the type of a tensor of `shape` and element type `elem` ("f32", "si8", ...)
MlirType tensorType(const std::vector<int64_t> &shape, const std::string &elem);

struct MlirWeight {
  std::string name;               // key in the weight file
  std::vector<int64_t> shape;     // from the load_weight result type
  std::string storage;            // "NONE", "INT8", "UINT32", ...
};

struct MlirModule {
  ModuleDesc module;
  std::string weight_file;            // filename attribute of tpu.weight_file ("" if none)
  std::vector<MlirWeight> weights;    // every tpu.load_weight
  std::string chipname;               // func attribute, "" if absent
};

MlirModule moduleFromMlir(const MlirFunc &func);

// One line per op: `type name quant param_type [shape] operands...`, then the returns;
// for tools and tests that only need to see what was understood.
std::string describeModule(const MlirModule &m);

}  // namespace tpuhip

// Calibration-table import and the INT8 quantisation pass over a parsed TPU-dialect
// function; tpuhip/quantize_pass.hpp says which reference code each part stands in for.
#include "tpuhip/quantize_pass.hpp"

#include <algorithm>
#include <cctype>
#include <cmath>
#include <fstream>
#include <functional>
#include <memory>
#include <numeric>
#include <set>
#include <sstream>
#include <stdexcept>

#include "tpuhip/quantize.hpp"
#include "tpuhip/tensor_file.hpp"

namespace tpuhip {

namespace {

[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error("quantize: " + msg); }

MlirAttr *find(MlirAttr &dict, const std::string &key) {
  for (auto &f : dict.fields)
    if (f.first == key) return &f.second;
  return nullptr;
}

MlirAttr &field(MlirAttr &dict, const std::string &key) {
  if (auto *a = find(dict, key)) return *a;
  dict.fields.emplace_back(key, MlirAttr());
  return dict.fields.back().second;
}

MlirAttr str_attr(const std::string &v) {
  MlirAttr a;
  a.kind = MlirAttr::String;
  a.str = v;
  return a;
}

MlirAttr f32_attr(float v) {
  MlirAttr a;
  a.kind = MlirAttr::Float;
  a.num = v;
  a.ty = "f32";
  return a;
}

std::string name_of(const MlirOp &o) {
  auto *n = o.attrs.get("name");
  return n && n->kind == MlirAttr::String ? n->str : std::string();
}

double num_attr(const MlirAttr &dict, const std::string &key, double dflt) {
  auto *a = dict.get(key);
  if (!a) return dflt;
  if (a->kind == MlirAttr::Int || a->kind == MlirAttr::Float || a->kind == MlirAttr::Bool) return a->num;
  return dflt;
}

bool is_reshape(const MlirOp &o) { return o.opname == "tpu.reshape"; }
bool is_weight(const MlirOp &o) { return o.opname == "tpu.load_weight"; }
bool is_none(const MlirOp &o) { return o.opname == "tpu.none"; }
bool is_tpu(const MlirOp &o) { return o.opname.compare(0, 4, "tpu.") == 0; }

// The function as a graph: who defines a value, how often it is used.
struct View {
  MlirFunc &f;
  std::map<std::string, int> def;    // SSA id -> index into f.ops
  std::map<std::string, int> uses;   // SSA id -> number of operand slots that name it

  explicit View(MlirFunc &func) : f(func) { rebuild(); }
  void rebuild() {
    def.clear();
    uses.clear();
    for (int i = 0; i < (int)f.ops.size(); ++i) {
      for (auto &r : f.ops[i].results) def[r] = i;
      for (auto &o : f.ops[i].operands) ++uses[o];
    }
  }
  MlirOp *producer(const std::string &id) {
    auto it = def.find(id);
    return it == def.end() ? nullptr : &f.ops[it->second];
  }
  // the op that answers for the quantisation of a value: a reshape hands every question
  // to its producer (TPUDialect.cpp, ReshapeOp::getOpQuant* / getOpQuantThreshold)
  MlirOp *quant_owner(MlirOp *o) {
    int guard = 0;
    while (o && is_reshape(*o) && !o->operands.empty() && ++guard < 1000) o = producer(o->operands[0]);
    return o;
  }
  bool has_quant(MlirOp *o) {
    o = quant_owner(o);
    if (!o) return false;
    auto *q = o->attrs.get("quant");
    return q && q->kind == MlirAttr::Dict;
  }
  MlirAttr &quant(MlirOp *o) {
    o = quant_owner(o);
    auto *q = o ? find(o->attrs, "quant") : nullptr;
    if (!q || q->kind != MlirAttr::Dict) fail("op '" + (o ? name_of(*o) : std::string("?")) + "' has no quant attribute");
    return *q;
  }
  float threshold(MlirOp *o) { return (float)num_attr(quant(o), "threshold", 0.0); }
  void set_threshold(MlirOp *o, float t) { field(quant(o), "threshold") = f32_attr(t); }
  std::string mode(MlirOp *o) {
    if (o && o->opname == "tpu.quant") {
      auto *to = o->attrs.get("to");
      return to && to->kind == MlirAttr::String ? to->str : "NONE";
    }
    if (!has_quant(o)) return "NONE";
    auto *m = quant(o).get("mode");
    return m && m->kind == MlirAttr::String ? m->str : "NONE";
  }
  void set_mode(MlirOp *o, const std::string &m) { field(quant(o), "mode") = str_attr(m); }
  void set_param_type(MlirOp *o, const std::string &t) { field(quant(o), "param_type") = str_attr(t); }
  float previous_threshold(MlirOp &o, size_t index = 0) {
    if (o.operands.size() <= index) fail("op '" + name_of(o) + "' has no operand " + std::to_string(index));
    MlirOp *p = producer(o.operands[index]);
    if (!p || !has_quant(p)) fail("operand " + std::to_string(index) + " of '" + name_of(o) + "' carries no threshold");
    return threshold(p);
  }
};

const std::set<std::string> kBackward = {"tpu.leaky_relu", "tpu.relu", "tpu.crop", "tpu.pool_max_2d"};
const std::set<std::string> kForward = {
    "tpu.abs", "tpu.copy", "tpu.crop", "tpu.leaky_relu", "tpu.relu", "tpu.pad", "tpu.pixelshuffle",
    "tpu.permute", "tpu.pool_max_2d", "tpu.reorg", "tpu.reverse", "tpu.reduce_max", "tpu.reduce_min",
    "tpu.shuffle_channel", "tpu.swap_channel", "tpu.tile", "tpu.upsample"};
// quantizeInt8BypassOps users within the INT8 interpreter's op set (QuantizeInt8.cpp:1606-1640)
const std::set<std::string> kBypass = {
    "tpu.crop", "tpu.dilate", "tpu.pad", "tpu.permute", "tpu.pixelshuffle", "tpu.pool_max_2d", "tpu.relu", "tpu.reorg",
    "tpu.reverse", "tpu.shuffle_channel", "tpu.swap_channel", "tpu.tile", "tpu.upsample"};
const std::map<std::string, LutKind> kLut = {
    {"tpu.sigmoid", LutKind::Sigmoid}, {"tpu.tanh", LutKind::TanH}, {"tpu.exp", LutKind::Exp},
    {"tpu.elu", LutKind::Elu}, {"tpu.swish", LutKind::Swish}, {"tpu.softplus", LutKind::SoftPlus},
    {"tpu.log", LutKind::Log}, {"tpu.pow", LutKind::Pow}, {"tpu.mish", LutKind::Mish}};

}  // namespace

CalibrationTable parseCalibrationTable(const std::string &text) {
  CalibrationTable t;
  std::istringstream in(text);
  std::string line;
  int lineno = 0;
  auto number = [](const std::string &w, float *out) {
    if (w.empty()) return false;
    // the reference's patterns accept [-0-9.e]+ only
    for (char c : w)
      if (!(std::isdigit((unsigned char)c) || c == '-' || c == '.' || c == 'e')) return false;
    char *end = nullptr;
    *out = std::strtof(w.c_str(), &end);
    return end && *end == 0;
  };
  while (std::getline(in, line)) {
    ++lineno;
    if (!line.empty() && line.back() == '\r') line.pop_back();
    std::istringstream iss(line);
    std::vector<std::string> w;
    for (std::string s; iss >> s;) w.push_back(s);
    if (w.empty() || line[0] == '#') continue;
    float v = 0;
    if (w.size() >= 2 && w[0] == "weight" && line.compare(0, 7, "weight ") == 0) {
      std::vector<float> th;
      for (size_t k = 2; k < w.size(); ++k) {
        if (!number(w[k], &v)) break;
        th.push_back(v);
      }
      t.weight_threshold[w[1]] = th;
    } else if (w.size() == 3 && w[0] == "bitwidth") {
      continue;
    } else if ((w.size() == 2 || w.size() == 4) && number(w[1], &v) &&
               (w.size() == 2 || (number(w[2], &v) && number(w[3], &v)))) {
      number(w[1], &v);
      t.threshold[w[0]] = v;
    } else {
      fail("calibration table line " + std::to_string(lineno) + " does not match the required format: '" + line + "'");
    }
  }
  return t;
}

std::vector<std::string> importCalibrationTable(MlirFunc &func, const CalibrationTable &table) {
  View g(func);
  std::vector<std::string> missing;
  for (auto &o : func.ops) {
    if (is_weight(o)) {
      auto it = table.weight_threshold.find(name_of(o));
      if (it != table.weight_threshold.end()) {
        MlirAttr arr;
        arr.kind = MlirAttr::Array;
        for (float v : it->second) arr.items.push_back(f32_attr(v));
        field(o.attrs, "threshold") = arr;
      }
      continue;
    }
    if (!is_tpu(o) || is_reshape(o) || !g.has_quant(&o) || name_of(o).empty()) continue;
    if (o.opname == "tpu.sigmoid" || o.opname == "tpu.tanh") {
      g.set_threshold(&o, 1.0f);
      g.set_param_type(&o, "THRESHOLD");
      continue;
    }
    auto it = table.threshold.find(name_of(o));
    if (it == table.threshold.end()) {
      missing.push_back(name_of(o));
      continue;
    }
    g.set_threshold(&o, it->second);
    g.set_param_type(&o, "THRESHOLD");
  }
  // each rule runs to its fixed point like a greedy pattern application; values only ever flow
  // one way along the edges of an acyclic graph, so that point does not depend on the order
  auto until_stable = [&](const std::function<bool(MlirOp &)> &rule) {
    for (size_t round = 0; round <= func.ops.size() + 1; ++round) {
      bool changed = false;
      for (auto &o : func.ops) changed = rule(o) || changed;
      if (!changed) return;
    }
  };
  // concat inputs (ImportCalibrationTable.cpp:152-178)
  until_stable([&](MlirOp &o) {
    if (o.opname != "tpu.concat" || !g.has_quant(&o)) return false;
    const float ty = g.threshold(&o);
    bool changed = false;
    const size_t n = o.operands.size() > 4 ? o.operands.size() - 4 : o.operands.size();
    for (size_t i = 0; i < n; ++i) {
      MlirOp *p = g.producer(o.operands[i]);
      if (!p || is_weight(*p) || is_none(*p)) break;
      if (!g.has_quant(p) || p->opname == "tpu.pool_max_2d") break;
      const float tx = g.threshold(p);
      if (g.uses[o.operands[i]] == 1 && tx != ty) {
        g.set_threshold(p, ty);
        changed = true;
      }
    }
    return changed;
  });
  // backward (:52-93)
  until_stable([&](MlirOp &o) {
    if (!kBackward.count(o.opname) || !g.has_quant(&o) || o.operands.empty()) return false;
    MlirOp *p = g.producer(o.operands[0]);
    if (!p || !g.has_quant(p)) return false;
    const float ty = g.threshold(&o), tx = g.threshold(p);
    if (tx == ty || g.uses[o.operands[0]] != 1) return false;
    g.set_threshold(p, ty);
    return true;
  });
  // mul_const: the result's threshold follows the input's (:133-150)
  until_stable([&](MlirOp &o) {
    if (o.opname != "tpu.mul_const" || !g.has_quant(&o) || o.operands.empty()) return false;
    MlirOp *p = g.producer(o.operands[0]);
    if (!p || !g.has_quant(p)) return false;
    const float c = (float)num_attr(o.attrs, "const_val", 0.0);
    const float tx = g.threshold(p), ty = g.threshold(&o);
    if (c == 0 || tx * std::abs(c) == ty) return false;
    g.set_threshold(&o, tx * std::abs(c));
    return true;
  });
  // forward (:184-208)
  until_stable([&](MlirOp &o) {
    if (!kForward.count(o.opname) || !g.has_quant(&o) || o.operands.empty()) return false;
    MlirOp *p = g.producer(o.operands[0]);
    if (!p || !g.has_quant(p)) return false;
    const float tx = g.threshold(p), ty = g.threshold(&o);
    if (tx == ty) return false;
    g.set_threshold(&o, tx);
    return true;
  });
  return missing;
}

namespace {

// Builds the quantised function op by op: new load_weight ops go in front of the op that
// uses them, values get fresh SSA names.
struct Quantizer {
  MlirFunc &func;
  WeightStore &weights;
  View g;
  std::vector<MlirOp> out;
  std::set<std::string> ids;
  std::string weight_file_id;
  MlirType weight_file_type;
  int counter = 0;

  Quantizer(MlirFunc &f, WeightStore &w) : func(f), weights(w), g(f) {
    for (auto &a : f.args) ids.insert(a.first);
    for (auto &o : f.ops) {
      for (auto &r : o.results) ids.insert(r);
      if (o.opname == "tpu.weight_file" && !o.results.empty() && !o.result_types.empty()) {
        weight_file_id = o.results[0];
        weight_file_type = o.result_types[0];
      }
    }
  }

  std::string fresh() {
    for (;;) {
      std::string id = "q" + std::to_string(counter++);
      if (ids.insert(id).second) return id;
    }
  }

  const WeightTensor &weight_of(MlirOp &o, size_t slot, const char *what) {
    MlirOp *p = slot < o.operands.size() ? g.producer(o.operands[slot]) : nullptr;
    if (!p || !is_weight(*p)) fail("op '" + name_of(o) + "': the " + what + " operand is not a tpu.load_weight");
    auto it = weights.find(name_of(*p));
    if (it == weights.end()) fail("op '" + name_of(o) + "': weight '" + name_of(*p) + "' is not in the weight file");
    return it->second;
  }
  bool operand_is_none(MlirOp &o, size_t slot) {
    MlirOp *p = slot < o.operands.size() ? g.producer(o.operands[slot]) : nullptr;
    return !p || is_none(*p);
  }

  // addWeightTensorAndUpdateWeightOp (TPUTensorSupport.cpp:206-256): the load_weight feeding
  // `slot` now loads a new tensor named after the old one
  void update_weight(MlirOp &o, size_t slot, const std::string &suffix, std::vector<float> data,
                     const std::vector<int64_t> &shape, const std::string &storage) {
    MlirOp *p = g.producer(o.operands[slot]);
    const std::string name = name_of(*p) + "_" + suffix;
    weights[name] = WeightTensor{shape, std::move(data)};
    // the op is already in `out` (it precedes its user); edit that copy too
    for (auto &w : out)
      if (is_weight(w) && !w.results.empty() && w.results[0] == o.operands[slot]) {
        field(w.attrs, "name") = str_attr(name);
        field(w.attrs, "storage") = str_attr(storage);
      }
    field(p->attrs, "name") = str_attr(name);
    field(p->attrs, "storage") = str_attr(storage);
  }

  // addWeightTensorAndCreateWeightOp (:277-311): "<op name>_<suffix>"
  void create_weight(MlirOp &o, size_t slot, const std::string &suffix, std::vector<float> data,
                     const std::vector<int64_t> &shape, const std::string &storage) {
    if (weight_file_id.empty()) {
      // a function without weights so far: give it the op every load_weight hangs on
      MlirOp wf;
      wf.opname = "tpu.weight_file";
      wf.results.push_back(fresh());
      wf.attrs.kind = MlirAttr::Dict;
      wf.attrs.fields.emplace_back("filename", str_attr(""));
      MlirType t;
      t.text = "memref<10xf32>";
      t.shaped = true;
      t.shape = {10};
      t.elem = "f32";
      wf.result_types.push_back(t);
      weight_file_id = wf.results[0];
      weight_file_type = t;
      out.insert(out.begin(), std::move(wf));
    }
    if (slot >= o.operands.size()) fail("op '" + name_of(o) + "' has no operand slot " + std::to_string(slot));
    const std::string name = name_of(o) + "_" + suffix;
    weights[name] = WeightTensor{shape, std::move(data)};
    MlirOp w;
    w.opname = "tpu.load_weight";
    w.results.push_back(fresh());
    w.operands.push_back(weight_file_id);
    w.attrs.kind = MlirAttr::Dict;
    w.attrs.fields.emplace_back("name", str_attr(name));
    w.attrs.fields.emplace_back("storage", str_attr(storage));
    w.operand_types.push_back(weight_file_type);
    w.result_types.push_back(tensorType(shape, "f32"));
    o.operands[slot] = w.results[0];
    o.operand_types[slot] = w.result_types[0];
    out.push_back(std::move(w));
  }

  void set_result_elem(MlirOp &o, const std::string &elem) {
    if (o.result_types.empty() || !o.result_types[0].shaped) return;
    o.result_types[0] = tensorType(o.result_types[0].shape, elem);
  }

  size_t data_inputs(MlirOp &o) {   // operands in front of the four quant operands
    if (o.operands.size() < 5) fail("op '" + name_of(o) + "': expected inputs followed by four quant operands");
    return o.operands.size() - 4;
  }

  // ---- per-op routines of QuantizeInt8.cpp -------------------------------------------
  void conv(MlirOp &o) {   // quantizeInt8ConvOps (:56-166)
    g.set_param_type(&o, "RSHIFT_AND_M_I32");
    if (o.operands.size() < 7) fail("conv '" + name_of(o) + "' needs 7 operands");
    const WeightTensor filter = weight_of(o, 1, "filter");
    int64_t oc = 0;
    if (filter.shape.size() == 4) oc = filter.shape[0];
    else if (filter.shape.size() == 5) oc = filter.shape[0] * filter.shape[1];
    else fail("conv '" + name_of(o) + "': filter must have 4 or 5 dimensions");
    const int64_t size = (int64_t)filter.data.size();
    if (oc <= 0 || size % oc) fail("conv '" + name_of(o) + "': bad filter shape");
    const bool has_bias = !operand_is_none(o, 2);
    WeightTensor bias;
    if (has_bias) {
      bias = weight_of(o, 2, "bias");
      if ((int64_t)bias.data.size() != oc) fail("conv '" + name_of(o) + "': bias size differs from the output channels");
    }
    std::vector<float> filter_threshold;
    if (auto *th = g.producer(o.operands[1])->attrs.get("threshold"))
      if (th->kind == MlirAttr::Array && (int64_t)th->items.size() == oc)
        for (auto &v : th->items) filter_threshold.push_back((float)v.num);
    const float tx = g.previous_threshold(o), ty = g.threshold(&o);
    std::vector<float> nf(size), nb(has_bias ? oc : 0), rs(oc), mu(oc);
    quantizeWeightInt8Multiplier(filter.data.data(), has_bias ? bias.data.data() : nullptr, oc, size / oc, ty, tx,
                                 nf.data(), has_bias ? nb.data() : nullptr, rs.data(), mu.data(), filter_threshold);
    const std::string suffix = std::to_string(ty) + "_quant";
    update_weight(o, 1, suffix, std::move(nf), filter.shape, "INT8");
    if (has_bias) update_weight(o, 2, suffix, std::move(nb), bias.shape, "INT32");
    create_weight(o, 5, "rshift", std::move(rs), {oc}, "UINT32");
    create_weight(o, 6, "multiplier", std::move(mu), {oc}, "UINT32");
  }

  void fully_connected(MlirOp &o) {   // quantizeInt8FullyConnectedOps (:171-249), batch 1
    g.set_param_type(&o, "RSHIFT_AND_M_I32");
    if (o.operands.size() < 7) fail("fully_connected '" + name_of(o) + "' needs 7 operands");
    const WeightTensor filter = weight_of(o, 1, "filter");
    if (filter.shape.size() != 2) fail("fully_connected '" + name_of(o) + "': only a 2-D filter (no batch) is supported");
    const int64_t n = filter.shape[0], k = filter.shape[1];
    const bool has_bias = !operand_is_none(o, 2);
    WeightTensor bias;
    if (has_bias) {
      bias = weight_of(o, 2, "bias");
      if ((int64_t)bias.data.size() != n) fail("fully_connected '" + name_of(o) + "': bias size differs from N");
    }
    const float tx = g.previous_threshold(o), ty = g.threshold(&o);
    std::vector<float> nf(filter.data.size()), nb(has_bias ? n : 0), rs(1), mu(1);
    quantizeWeightInt8ForFC(filter.data.data(), has_bias ? bias.data.data() : nullptr, 1, n, k, ty, tx, nf.data(),
                            has_bias ? nb.data() : nullptr, rs.data(), mu.data());
    update_weight(o, 1, "quant", std::move(nf), filter.shape, "INT8");
    if (has_bias) update_weight(o, 2, "quant", std::move(nb), bias.shape, "INT32");
    create_weight(o, 5, "rshift", std::move(rs), {1}, "NONE");
    create_weight(o, 6, "multiplier", std::move(mu), {1}, "NONE");
  }

  void rescale(MlirOp &o) {   // quantizeInt8RescaleNoWeightOps (:669-854)
    g.set_param_type(&o, "RSHIFT_AND_M_I8");
    const float ty = g.threshold(&o);
    size_t n = data_inputs(o);
    if (o.opname == "tpu.clip") {
      n = 1;
      // the bounds in output steps, truncated like the reference's int conversion
      const int lo = (int)(num_attr(o.attrs, "min", 0.0) * 127.0 / ty);
      const int hi = (int)(num_attr(o.attrs, "max", 0.0) * 127.0 / ty);
      field(o.attrs, "min") = f32_attr((float)lo);
      field(o.attrs, "max") = f32_attr((float)hi);
    }
    std::vector<float> tx(n);
    bool bypass = true;
    for (size_t i = 0; i < n; ++i) {
      tx[i] = g.previous_threshold(o, i);
      if (std::fabs(ty - tx[i]) > 1e-5f) bypass = false;
    }
    const bool always = o.opname == "tpu.pool_avg_2d" || o.opname == "tpu.eltwise_max" ||
                        o.opname == "tpu.eltwise_min" || o.opname == "tpu.eltwise_add";
    if (bypass && !always) {
      g.set_param_type(&o, "NONE");   // rshift and multiplier stay none: no rescaling
      return;
    }
    std::vector<float> coeff;
    if (o.opname == "tpu.eltwise_add")
      if (auto *c = o.attrs.get("coeff"))
        if (c->kind == MlirAttr::Array && c->items.size() == n)
          for (auto &v : c->items) coeff.push_back((float)v.num);
    int divisor = 1;
    if (o.opname == "tpu.pool_avg_2d") {
      auto *p = find(o.attrs, "param");
      if (!p || p->kind != MlirAttr::Dict) fail("pool_avg_2d '" + name_of(o) + "' has no param attribute");
      const int kh = (int)num_attr(*p, "kernel_h", 1);
      int kw = (int)num_attr(*p, "kernel_w", 1);
      if (kw == 0) kw = 1;
      divisor = kh * kw;
      MlirAttr yes;
      yes.kind = MlirAttr::Bool;
      yes.num = 1;
      field(*p, "count_include_pad") = yes;   // the INT8 form only knows this mode
    }
    std::vector<float> rs(1), mu(n);
    quantizeRescaleNoWeight(tx, ty, coeff, divisor, rs.data(), mu.data());
    const size_t slot = o.opname == "tpu.clip" ? o.operands.size() - 2 : n + 2;
    create_weight(o, slot, "rshift", std::move(rs), {1}, "NONE");
    create_weight(o, slot + 1, "multiplier", std::move(mu), {(int64_t)n}, "NONE");
  }

  void multiply(MlirOp &o) {   // quantizeInt8MultiplyOps (:1108-1170)
    g.set_param_type(&o, "RSHIFT_AND_M_I32");
    const size_t n = data_inputs(o);
    for (size_t i = 0; i < n; ++i) {
      MlirOp *p = g.producer(o.operands[i]);
      if (p && is_weight(*p)) fail("op '" + name_of(o) + "': a constant operand is not supported in INT8 (the reference runs it in BF16)");
    }
    const float ty = g.threshold(&o);
    double prod = 1.0;
    for (size_t i = 0; i < n; ++i) prod *= g.previous_threshold(o, i);
    const float qscale = (float)(prod / ty / 127.0);
    std::vector<float> rs(1, 0.0f), mu(1, 0.0f);
    if (std::abs(qscale - 1.0f) > 1e-5) {
      uint32_t m = 0;
      rs[0] = (float)findRShiftAndMultiplierFromQScale(qscale, &m, true);
      mu[0] = (float)m;
    }
    create_weight(o, n + 2, "rshift", std::move(rs), {1}, "NONE");
    create_weight(o, n + 3, "multiplier", std::move(mu), {1}, "NONE");
  }

  void concat(MlirOp &o) {   // quantizeInt8ConcatOps (:856-896)
    g.set_param_type(&o, "RSHIFT_AND_M_I8");
    const size_t n = data_inputs(o);
    const float ty = g.threshold(&o);
    std::vector<float> rs(n, 0.0f), mu(n, 1.0f);
    for (size_t i = 0; i < n; ++i) {
      const float tx = g.previous_threshold(o, i);
      float qscale = tx / ty;
      if (std::fabs(ty - tx) <= 1e-5) qscale = 1.0f;
      if (qscale != 1.0f) {
        uint32_t m = 0;
        rs[i] = (float)findRShiftAndMultiplierFromQScale(qscale, &m);
        mu[i] = (float)m;
      }
    }
    create_weight(o, n + 2, "rshift", std::move(rs), {(int64_t)n}, "NONE");
    create_weight(o, n + 3, "multiplier", std::move(mu), {(int64_t)n}, "NONE");
  }

  void leaky_relu(MlirOp &o) {   // quantizeInt8LeakyReluOps (:349-429)
    g.set_param_type(&o, "RSHIFT_AND_M_I8");
    if (o.operands.size() < 9) fail("leaky_relu '" + name_of(o) + "' needs 9 operands");
    float q[4];
    quantizeLeakyRelu((float)num_attr(o.attrs, "negative_slope", 0.0), g.previous_threshold(o), g.threshold(&o), q);
    static const char *names[4] = {"rshift_pos", "multiplier_pos", "rshift_neg", "multiplier_neg"};
    for (int i = 0; i < 4; ++i) create_weight(o, 5 + i, names[i], {q[i]}, {1}, "NONE");
  }

  void prelu(MlirOp &o) {   // quantizeInt8PReluOps (:433-525)
    g.set_param_type(&o, "RSHIFT_AND_M_I8");
    if (o.operands.size() < 9) fail("prelu '" + name_of(o) + "' needs 9 operands");
    const WeightTensor slope = weight_of(o, 1, "slope");
    if (slope.shape.size() < 2 || (int64_t)slope.data.size() < slope.shape[1] || slope.shape[1] < 1)
      fail("prelu '" + name_of(o) + "': the slope must be shaped 1 x c x 1 x 1");
    const int c = (int)slope.shape[1];
    const float tx = g.previous_threshold(o), ty = g.threshold(&o);
    float rshift_pos = 0, multiplier_pos = 1.0f;
    const double qscale_pos = tx / ty;
    if (!(std::fabs(tx - ty) < 1e-5 * std::min(tx, ty))) {
      uint32_t m = 0;
      rshift_pos = (float)findRShiftAndMultiplierFromQScale(qscale_pos, &m, false);
      multiplier_pos = (float)m;
    }
    double max_neg = std::fabs(qscale_pos * slope.data[0]);
    for (int i = 1; i < c; ++i) max_neg = std::max(max_neg, std::fabs(qscale_pos * slope.data[i]));
    uint32_t m_neg = 0;
    const float rshift_neg = (float)findRShiftAndMultiplierFromQScale(max_neg, &m_neg, false);
    std::vector<float> q(slope.data.size(), 0.0f);
    for (int i = 0; i < c; ++i) {
      // quantizeFilterRShift (QuantizationArithmetic.cpp:399-404), saturateInt8 = floor(x + 0.5) clamped
      const double factor = (tx / ty) * (1 << (uint32_t)rshift_neg);
      const float qf = (float)(slope.data[i] * factor);
      q[i] = (float)std::max(-128.0, std::min(127.0, std::floor(qf + 0.5)));   // the sum in double, like the reference
    }
    update_weight(o, 1, "negative_slope", std::move(q), slope.shape, "INT8");
    create_weight(o, 6, "rshift_pos", {rshift_pos}, {1}, "NONE");
    create_weight(o, 7, "multiplier_pos", {multiplier_pos}, {1}, "NONE");
    create_weight(o, 8, "rshift_neg", {rshift_neg}, {1}, "NONE");
  }

  void lut(MlirOp &o, LutKind kind) {   // quantizeInt8LutOps (:531-621)
    if (o.operands.size() < 2) fail("op '" + name_of(o) + "' has no table operand");
    float t256[256];
    const bool has_scale = kind == LutKind::Sigmoid || kind == LutKind::Exp || kind == LutKind::SoftPlus;
    quantizeLutTable(kind, g.previous_threshold(o), g.threshold(&o),
                     has_scale ? (float)num_attr(o.attrs, "scale", 1.0) : 1.0f,
                     has_scale ? (float)num_attr(o.attrs, "bias", 0.0) : 0.0f,
                     (float)num_attr(o.attrs, "coeff", 0.0), t256);
    // one copy of the table per lane of the chip the reference targets (32 lanes)
    const int lanes = 32;
    std::vector<float> table((size_t)lanes * 256);
    for (int l = 0; l < lanes; ++l) std::copy(t256, t256 + 256, table.begin() + (size_t)l * 256);
    create_weight(o, 1, "y0_table", std::move(table), {1, lanes, 16, 16}, "INT8");
  }

  // quantize_fraction (:251-262): x / y as an integer over 2^rshift, the largest shift (up to
  // 15) whose power of two stays below 256 * y / x
  static void quantize_fraction(float x, float y, int &rshift_width, int &x_quantized) {
    const float y_ceiling = 256.0 / x * y;
    rshift_width = 0;
    float y_quantized = 1.0;
    while ((y_quantized * 2) < y_ceiling && rshift_width < 15) {
      rshift_width += 1;
      y_quantized = (float)(1 << rshift_width);
    }
    x_quantized = (int)std::floor((x / y) * y_quantized + 0.5);
  }

  void lrn(MlirOp &o) {   // quantizeInt8LrnOps (:264-347)
    if (o.operands.size() < 3) fail("lrn '" + name_of(o) + "' needs the two table operands");
    const uint32_t local_size = (uint32_t)num_attr(o.attrs, "local_size", 0);
    const float alpha = (float)num_attr(o.attrs, "alpha", 0), beta = (float)num_attr(o.attrs, "beta", 0),
                k = (float)num_attr(o.attrs, "k", 0);
    auto *parts = o.attrs.get("threshold_parts");
    if (local_size == 0 || !parts || parts->kind != MlirAttr::Array || parts->items.size() < 3)
      fail("lrn '" + name_of(o) + "': local_size and the three threshold_parts (squares, their sum, the scale) are needed");
    const float sq_thy = (float)parts->items[0].num, sumsq_thy = (float)parts->items[1].num,
                scale_thy = (float)parts->items[2].num;
    const float threshold_x = g.previous_threshold(o), threshold_y = g.threshold(&o);
    int quant_x0 = 0, sum_rshift = 0, quant_x1 = 0, lrn_rshift = 0;
    quantize_fraction(sq_thy, sumsq_thy, sum_rshift, quant_x0);
    quantize_fraction(threshold_x * scale_thy, threshold_y * 256.0, lrn_rshift, quant_x1);
    auto i32 = [](int v) {
      MlirAttr a;
      a.kind = MlirAttr::Int;
      a.num = v;
      a.ty = "i32";
      return a;
    };
    field(o.attrs, "sum_rshift") = i32(sum_rshift);
    field(o.attrs, "quant_data0") = i32(quant_x0);
    field(o.attrs, "lrn_rshift") = i32(lrn_rshift);
    field(o.attrs, "quant_data1") = i32(quant_x1);
    const int lanes = 32;
    std::vector<float> sq_table((size_t)lanes * 256), power_table((size_t)lanes * 256);
    for (int idx = 0; idx < 256; ++idx) {
      // the mix of float and double below is the reference's
      float lut_input = threshold_x / 128.0 * idx;
      float lut_output = std::pow(lut_input, 2) * 256.0 / sq_thy;
      lut_output = lut_output * alpha / local_size;
      lut_output = std::floor(lut_output + 0.5);
      if (lut_output > 255.0) lut_output = 255.0;
      for (int n = 0; n < lanes; ++n) sq_table[(size_t)n * 256 + idx] = lut_output;
      lut_input = (float)idx / (256.0 / sumsq_thy);
      lut_output = std::pow(lut_input + k, -beta);
      lut_output = lut_output * (256.0 / scale_thy);
      lut_output = std::floor(lut_output + 0.5);
      if (lut_output > 255.0) lut_output = 255.0;
      for (int n = 0; n < lanes; ++n) power_table[(size_t)n * 256 + idx] = lut_output;
    }
    create_weight(o, 1, "sq_gen_weight", std::move(sq_table), {1, lanes, 16, 16}, "UINT8");
    create_weight(o, 2, "power_gen_weight", std::move(power_table), {1, lanes, 16, 16}, "UINT8");
  }

  void bypass(MlirOp &o) {   // quantizeInt8BypassOps (:1206-1248)
    g.set_param_type(&o, "NONE");
    const float tx = g.previous_threshold(o), ty = g.threshold(&o);
    if (tx - ty > 0.001f)
      fail("op '" + name_of(o) + "' (" + o.opname + ") passes its input through but the thresholds differ: x = " +
           std::to_string(tx) + ", y = " + std::to_string(ty));
  }

  void quantize_op(MlirOp &o) {
    const std::string &t = o.opname;
    g.set_mode(&o, "INT8");
    if (t == "tpu.conv_2d" || t == "tpu.deconv_2d") conv(o);
    else if (t == "tpu.fully_connected") fully_connected(o);
    else if (t == "tpu.eltwise_add" || t == "tpu.eltwise_max" || t == "tpu.eltwise_min" ||
             t == "tpu.broadcast_add" || t == "tpu.broadcast_sub" || t == "tpu.pool_avg_2d" || t == "tpu.clip") {
      if (t == "tpu.eltwise_add")
        for (size_t i = 0; i < 2 && i < o.operands.size(); ++i) {
          MlirOp *p = g.producer(o.operands[i]);
          if (p && is_weight(*p)) fail("op '" + name_of(o) + "': a constant operand is not supported in INT8");
        }
      rescale(o);
    } else if (t == "tpu.eltwise_mul" || t == "tpu.broadcast_mul") multiply(o);
    else if (t == "tpu.concat") concat(o);
    else if (t == "tpu.leaky_relu") leaky_relu(o);
    else if (t == "tpu.prelu") prelu(o);
    else if (t == "tpu.lrn") lrn(o);
    else if (t == "tpu.mul_const") {   // quantizeInt8MulConstOps (:1178-1197): only the sign is left
      const float c = (float)num_attr(o.attrs, "const_val", 0.0);
      field(o.attrs, "const_val") = f32_attr(c > 0.0f ? 1.0f : c < 0.0f ? -1.0f : 0.0f);
    } else if (t == "tpu.reflection_pad") {
      // ReflectionPadOp::quantizeInt8 (:1389-1414): one K x K anti-diagonal 0/1 matrix per pad
      // (what the TPU multiplies the edge columns by to mirror them; the interpreter does not
      // read them), named <op>_select_<i>, in operand slots 1 and 2
      auto *pads = o.attrs.get("pads");
      if (!pads || pads->kind != MlirAttr::Array || pads->items.size() != 2)
        fail("reflection_pad '" + name_of(o) + "': pads must hold two numbers");
      for (size_t i = 0; i < 2; ++i) {
        const int64_t K = (int64_t)pads->items[i].num;
        if (K < 0) fail("reflection_pad '" + name_of(o) + "': negative pad");
        std::vector<float> select((size_t)(K * K), 0.0f);
        for (int64_t r = 0; r < K; ++r) select[(size_t)(r * K + (K - r - 1))] = 1.0f;
        create_weight(o, i + 1, "select_" + std::to_string(i), std::move(select), {K, K}, "INT8");
      }
    } else if (kLut.count(t)) lut(o, kLut.at(t));
    else if (kBypass.count(t)) bypass(o);
    else fail("op '" + name_of(o) + "': no INT8 quantisation for " + t);
    set_result_elem(o, "si8");
  }

  // ---- insertQuantOp (Quantization.cpp:99-255) -----------------------------------------
  // `o` is the op being emitted; its operands may be replaced by new tpu.quant results
  std::map<std::string, std::string> quant_of;   // "<value id>|<quant op name>" -> result id

  void insert_quant(MlirOp &o) {
    std::string curr;
    if (is_reshape(o)) {
      MlirOp *p = o.operands.empty() ? nullptr : g.producer(o.operands[0]);
      if (!p || p->opname != "tpu.input") return;
      // the single user decides
      MlirOp *next = nullptr;
      int users = 0;
      for (auto &u : func.ops)
        for (auto &opd : u.operands)
          if (!o.results.empty() && opd == o.results[0]) { next = &u; ++users; }
      if (users != 1 || !next || is_reshape(*next)) return;
      curr = next->opname == "std.return" ? "NONE" : g.mode(next);
    } else {
      curr = o.opname == "std.return" ? "NONE" : g.mode(&o);
    }
    for (size_t i = 0; i < o.operands.size(); ++i) {
      MlirOp *prev = g.producer(o.operands[i]);
      if (!prev) fail("operand " + std::to_string(i) + " of '" + name_of(o) + "' is a function argument: expected a tpu.input in front");
      if (prev->opname == "tpu.quant" || is_weight(*prev) || is_none(*prev) || prev->opname == "tpu.weight_file") continue;
      if (is_reshape(*prev)) {
        MlirOp *pp = prev->operands.empty() ? nullptr : g.producer(prev->operands[0]);
        if (pp && pp->opname == "tpu.quant") continue;
      }
      const std::string prev_name = name_of(*prev);
      MlirOp *owner = g.quant_owner(prev);
      const std::string prev_quant = g.mode(owner);
      if (curr == prev_quant) continue;
      const bool curr8 = curr == "INT8" || curr == "UINT8", prev8 = prev_quant == "INT8" || prev_quant == "UINT8";
      if (curr8 && prev8) continue;
      float scale = 1.0f;
      std::string name;
      if (curr8) {
        scale = (curr == "INT8" ? 128 : 256) / g.threshold(owner);
        name = prev_name + "_quant_i8";
      } else if (prev8) {
        scale = g.threshold(owner) / (prev_quant == "INT8" ? 128 : 256);
        name = prev_name + (curr == "BF16" ? "_dequant_bf16" : "_dequant");
      } else {
        fail("op '" + name_of(o) + "': only fp32 <-> INT8 conversions are inserted (" + prev_quant + " -> " + curr + ")");
      }
      const std::string key = o.operands[i] + "|" + name;
      auto it = quant_of.find(key);
      if (it == quant_of.end()) {
        MlirOp q;
        q.opname = "tpu.quant";
        q.results.push_back(fresh());
        q.operands.push_back(o.operands[i]);
        q.operand_types.push_back(o.operand_types[i]);
        q.attrs.kind = MlirAttr::Dict;
        q.attrs.fields.emplace_back("from", str_attr(prev_quant));
        q.attrs.fields.emplace_back("to", str_attr(curr));
        q.attrs.fields.emplace_back("scale", f32_attr(scale));
        q.attrs.fields.emplace_back("name", str_attr(name));
        const MlirType &src = o.operand_types[i];
        q.result_types.push_back(src.shaped ? tensorType(src.shape, curr == "INT8" ? "si8" : "f32") : src);
        it = quant_of.emplace(key, q.results[0]).first;
        out.push_back(std::move(q));
        quant_types[it->second] = out.back().result_types[0];
      }
      o.operands[i] = it->second;
      o.operand_types[i] = quant_types[it->second];
      if (is_reshape(o)) field(o.attrs, "name") = str_attr(name_of(o) + "_quant");
    }
  }
  std::map<std::string, MlirType> quant_types;

  void run() {
    // 1. quantise every op (the walk of Quantization.cpp:697-745); result types change here,
    //    so remember them for the operand types of the users
    std::map<std::string, MlirType> new_type;
    std::vector<MlirOp> staged;
    for (auto &o : func.ops) {
      const bool skip = !is_tpu(o) || o.opname == "tpu.input" || o.opname == "tpu.quant" || is_reshape(o) ||
                        is_weight(o) || is_none(o) || o.opname == "tpu.weight_file";
      if (!skip) {
        if (!g.has_quant(&o)) fail("op '" + name_of(o) + "' (" + o.opname + ") has no quant attribute");
        quantize_op(o);
      }
      out.push_back(o);
    }
    // the ops created so far sit in `out` in front of their users; make that the function
    func.ops = out;
    out.clear();
    g.rebuild();
    for (auto &o : func.ops)
      for (size_t k = 0; k < o.results.size() && k < o.result_types.size(); ++k) new_type[o.results[k]] = o.result_types[k];
    auto refresh_operand_types = [&](MlirOp &o) {
      for (size_t i = 0; i < o.operands.size(); ++i) {
        auto it = new_type.find(o.operands[i]);
        if (it != new_type.end()) o.operand_types[i] = it->second;
      }
    };
    // a reshape keeps the element type of what it reshapes (Quantization.cpp:764-772)
    for (auto &o : func.ops) {
      refresh_operand_types(o);
      if (is_reshape(o) && !o.operand_types.empty() && o.operand_types[0].shaped && !o.result_types.empty() &&
          o.result_types[0].shaped) {
        o.result_types[0] = tensorType(o.result_types[0].shape, o.operand_types[0].elem);
        new_type[o.results[0]] = o.result_types[0];
      }
    }
    // 2. tpu.quant where the modes differ (the walk of :748-760)
    std::vector<MlirOp> ops = func.ops;
    for (auto &o : ops) {
      const bool skip = (!is_tpu(o) && o.opname != "std.return") || o.opname == "tpu.input" ||
                        o.opname == "tpu.weight_file" || is_weight(o) || is_none(o);
      if (!skip) insert_quant(o);
      out.push_back(o);
    }
    func.ops = out;
    out.clear();
    g.rebuild();
    new_type.clear();
    for (auto &o : func.ops)
      for (size_t k = 0; k < o.results.size() && k < o.result_types.size(); ++k) new_type[o.results[k]] = o.result_types[k];
    for (auto &o : func.ops) {
      refresh_operand_types(o);
      if (is_reshape(o) && !o.operand_types.empty() && o.operand_types[0].shaped && !o.result_types.empty() &&
          o.result_types[0].shaped) {
        o.result_types[0] = tensorType(o.result_types[0].shape, o.operand_types[0].elem);
        new_type[o.results[0]] = o.result_types[0];
      }
      if (o.opname == "std.return") func.results = o.operand_types;
    }
  }
};

std::string dir_of(const std::string &path) {
  const size_t k = path.find_last_of('/');
  return k == std::string::npos ? std::string() : path.substr(0, k + 1);
}

std::string base_of(const std::string &path) {
  const size_t k = path.find_last_of('/');
  return k == std::string::npos ? path : path.substr(k + 1);
}

std::string read_text(const std::string &path) {
  std::ifstream f(path, std::ios::binary);
  if (!f.good()) throw std::runtime_error("cannot open '" + path + "'");
  std::ostringstream ss;
  ss << f.rdbuf();
  return ss.str();
}

}  // namespace

void quantizeInt8(MlirFunc &func, WeightStore &weights) {
  Quantizer q(func, weights);
  q.run();
}

WeightStore readWeights(const MlirFunc &func, const std::string &mlir_path) {
  WeightStore store;
  std::string file;
  for (auto &o : func.ops)
    if (o.opname == "tpu.weight_file")
      if (auto *fn = o.attrs.get("filename"))
        if (fn->kind == MlirAttr::String) file = fn->str;
  std::unique_ptr<TensorFile> tf;
  for (auto &o : func.ops) {
    if (!is_weight(o)) continue;
    if (!tf) {
      if (file.empty()) fail(mlir_path + ": tpu.load_weight without a tpu.weight_file");
      std::string path = file;
      if (!std::ifstream(path, std::ios::binary).good() && path[0] != '/') path = dir_of(mlir_path) + file;
      tf.reset(new TensorFile(path, true));
    }
    const std::string name = name_of(o);
    if (o.result_types.empty() || !o.result_types[0].shaped) fail("weight '" + name + "' has no tensor type");
    WeightTensor w;
    w.shape = o.result_types[0].shape;
    size_t count = 1;
    for (auto d : w.shape) {
      if (d < 0) fail("weight '" + name + "': dynamic shape");
      count *= (size_t)d;
    }
    w.data.resize(count);
    if (!tf->readTensor(name, w.data.data(), count))
      fail("weight '" + name + "' is missing from " + tf->path() + " or is not float32 x " + std::to_string(count));
    store[name] = std::move(w);
  }
  return store;
}

std::vector<std::string> quantizeFiles(const std::string &in_mlir, const std::string &calibration_table,
                                       const std::string &out_mlir, std::string out_weights) {
  MlirFunc func = parseMlirText(read_text(in_mlir));
  WeightStore weights = readWeights(func, in_mlir);
  const CalibrationTable table = parseCalibrationTable(read_text(calibration_table));
  std::vector<std::string> missing = importCalibrationTable(func, table);
  quantizeInt8(func, weights);
  if (out_weights.empty()) {
    const size_t dot = out_mlir.find_last_of('.');
    const size_t slash = out_mlir.find_last_of('/');
    const bool has_ext = dot != std::string::npos && (slash == std::string::npos || dot > slash);
    out_weights = (has_ext ? out_mlir.substr(0, dot) : out_mlir) + "_weights.npz";
  }
  // only the tensors the quantised function still loads
  TensorFile tf(out_weights, false, true);
  for (auto &o : func.ops) {
    if (o.opname == "tpu.weight_file") field(o.attrs, "filename") = str_attr(base_of(out_weights));
    if (!is_weight(o)) continue;
    const std::string name = name_of(o);
    auto it = weights.find(name);
    if (it == weights.end()) fail("weight '" + name + "' vanished");
    if (!tf.find(name)) tf.addTensor(name, it->second.data.data(), it->second.shape);
  }
  tf.keep();
  std::ofstream f(out_mlir, std::ios::binary);
  if (!f.good()) throw std::runtime_error("cannot write '" + out_mlir + "'");
  f << printMlir(func);
  return missing;
}

}  // namespace tpuhip

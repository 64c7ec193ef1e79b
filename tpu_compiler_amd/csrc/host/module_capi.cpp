// C ABI over the C++ ModuleInterpreter: exceptions become status codes.
#include <cstdarg>
#include <cstring>

#include "tpuhip/interpreter.hpp"

namespace tpuhip {
int set_error(int status, const char *fmt, ...);
}

struct tpuhip_module {
  std::unique_ptr<tpuhip::ModuleInterpreter> interp;
  tpuhip::ModuleDesc desc;
  std::vector<std::string> tensor_names;
  std::string scratch;
};

using namespace tpuhip;

#define GUARD(m, body)                                                        \
  if (!(m)) return set_error(TPUHIP_ERR_INVALID, "%s: NULL module", __func__); \
  try {                                                                       \
    body;                                                                     \
  } catch (const std::exception &e) {                                         \
    return set_error(TPUHIP_ERR_INVALID, "%s", e.what());                     \
  }                                                                           \
  return TPUHIP_OK;

extern "C" {

int tpuhip_module_create(int device, int max_batch, tpuhip_module **out) {
  if (!out) return set_error(TPUHIP_ERR_INVALID, "tpuhip_module_create: out is NULL");
  try {
    auto *m = new tpuhip_module();
    m->interp.reset(new ModuleInterpreter(max_batch, device));
    *out = m;
  } catch (const std::exception &e) {
    return set_error(TPUHIP_ERR_INVALID, "%s", e.what());
  }
  return TPUHIP_OK;
}

int tpuhip_module_destroy(tpuhip_module *m) {
  delete m;
  return TPUHIP_OK;
}

int tpuhip_module_set_weight(tpuhip_module *m, const char *name, const float *data, size_t count) {
  GUARD(m, {
    if (!name || (!data && count)) throw std::runtime_error("set_weight: NULL argument");
    m->interp->updateWeightMap(name, data, count);
  })
}

int tpuhip_module_clear_ops(tpuhip_module *m) {
  GUARD(m, {
    m->desc.ops.clear();
    m->desc.returns.clear();
  })
}

int tpuhip_module_add_op(tpuhip_module *m, const tpuhip_op_desc *op) {
  GUARD(m, {
    if (!op || !op->type || !op->name) throw std::runtime_error("add_op: NULL argument");
    OpDesc d;
    d.type = op->type;
    d.name = op->name;
    if (op->quant) d.quant = op->quant;
    if (op->param_type) d.param_type = op->param_type;
    for (int i = 0; i < op->ndim; ++i) d.shape.push_back(op->shape[i]);
    for (int i = 0; i < op->n_operands; ++i) d.operands.push_back(op->operands[i] ? op->operands[i] : "");
    for (int i = 0; i < op->n_attrs; ++i) d.attrs[op->attr_keys[i]] = op->attr_values[i];
    m->desc.ops.push_back(std::move(d));
  })
}

int tpuhip_module_set_returns(tpuhip_module *m, const char *const *names, int n) {
  GUARD(m, {
    m->desc.returns.clear();
    for (int i = 0; i < n; ++i) m->desc.returns.push_back(names[i]);
  })
}

int tpuhip_module_set_option(tpuhip_module *m, const char *key, int value) {
  GUARD(m, {
    const std::string k = key ? key : "";
    if (k == "fuse_eltwise")
      m->interp->fuse_eltwise = value != 0;
    else if (k == "keep_all_tensors")
      m->interp->keep_all_tensors = value != 0;
    else
      throw std::runtime_error("tpuhip_module_set_option: unknown option '" + k + "'");
  })
}

int tpuhip_module_load(tpuhip_module *m, const char *target_op) {
  GUARD(m, {
    m->interp->loadModule(m->desc, target_op ? target_op : "");
    m->tensor_names = m->interp->getAllTensorName();
  })
}

int tpuhip_module_set_tensor(tpuhip_module *m, const char *name, const float *data, size_t count,
                             int bidx) {
  GUARD(m, {
    if (!name || !data) throw std::runtime_error("set_tensor: NULL argument");
    std::string n(name);
    std::vector<float> v(data, data + count);
    m->interp->setTensor(n, v, bidx);
  })
}

int tpuhip_module_get_tensor(tpuhip_module *m, const char *name, float *dst, size_t count,
                             int bidx) {
  GUARD(m, {
    if (!name || !dst) throw std::runtime_error("get_tensor: NULL argument");
    std::string n(name);
    auto t = m->interp->getTensor(n, bidx);
    if (t->size() != count) throw std::runtime_error("get_tensor: size mismatch");
    memcpy(dst, t->data(), count * sizeof(float));
  })
}

int tpuhip_module_get_tensor_i8(tpuhip_module *m, const char *name, int8_t *dst, size_t count,
                                int bidx) {
  GUARD(m, {
    if (!name || !dst) throw std::runtime_error("get_tensor_i8: NULL argument");
    m->interp->getTensorI8(name, dst, count, bidx);
  })
}

int tpuhip_module_invoke(tpuhip_module *m, int bidx) { GUARD(m, m->interp->invoke(bidx)) }

int tpuhip_module_invoke_to(tpuhip_module *m, const char *name, int bidx) {
  GUARD(m, m->interp->invokeTo(name ? name : "", bidx))
}

int tpuhip_module_fast_invoke_all_batch(tpuhip_module *m, const char *name, int batch) {
  GUARD(m, m->interp->fastInvokeAllBatch(name ? name : "", batch))
}

int tpuhip_module_sync(tpuhip_module *m) { GUARD(m, m->interp->sync()) }

int tpuhip_module_tensor_shape(tpuhip_module *m, const char *name, int64_t *dims8, int *ndim) {
  GUARD(m, {
    if (!name || !dims8 || !ndim) throw std::runtime_error("tensor_shape: NULL argument");
    std::string n(name);
    auto s = m->interp->getTensorShape(n);
    if (s.size() > 8) throw std::runtime_error("tensor_shape: rank > 8");
    *ndim = (int)s.size();
    for (size_t i = 0; i < s.size(); ++i) dims8[i] = s[i];
  })
}

const char *tpuhip_module_tensor_dtype(tpuhip_module *m, const char *name) {
  if (!m || !name) return nullptr;
  try {
    std::string n(name);
    m->scratch = m->interp->getDataType(n);
    return m->scratch.c_str();
  } catch (const std::exception &e) {
    set_error(TPUHIP_ERR_INVALID, "%s", e.what());
    return nullptr;
  }
}

int tpuhip_module_num_tensors(tpuhip_module *m) { return m ? (int)m->tensor_names.size() : 0; }
const char *tpuhip_module_tensor_name(tpuhip_module *m, int i) {
  return (m && i >= 0 && i < (int)m->tensor_names.size()) ? m->tensor_names[i].c_str() : nullptr;
}
int tpuhip_module_num_inputs(tpuhip_module *m) { return m ? (int)m->interp->input_details.size() : 0; }
const char *tpuhip_module_input_name(tpuhip_module *m, int i) {
  return (m && i >= 0 && i < (int)m->interp->input_details.size())
             ? m->interp->input_details[i].first.c_str() : nullptr;
}
int tpuhip_module_num_outputs(tpuhip_module *m) { return m ? (int)m->interp->output_details.size() : 0; }
const char *tpuhip_module_output_name(tpuhip_module *m, int i) {
  return (m && i >= 0 && i < (int)m->interp->output_details.size())
             ? m->interp->output_details[i].c_str() : nullptr;
}

int tpuhip_module_num_kernels(tpuhip_module *m) { return m ? (int)m->interp->kernels().size() : 0; }

static CPUOpKernel *kernel_at(tpuhip_module *m, int i) {
  if (!m || i < 0) return nullptr;
  for (auto &k : m->interp->kernels())
    if (i-- == 0) return k.get();
  return nullptr;
}

const char *tpuhip_module_kernel_name(tpuhip_module *m, int i) {
  auto *k = kernel_at(m, i);
  return k ? k->name.c_str() : nullptr;
}

const char *tpuhip_module_kernel_algo(tpuhip_module *m, int i) {
  auto *k = kernel_at(m, i);
  if (!k) return nullptr;
  if (auto *c = dynamic_cast<Conv2DOpKernel *>(k)) return c->algo_name();
  if (dynamic_cast<FullyConnectedOpKernel *>(k)) return "fc";
  return "";
}

int tpuhip_module_time_kernels(tpuhip_module *m, int bidx, int iters, float *ms, int capacity) {
  GUARD(m, {
    auto t = m->interp->timeKernels(bidx, iters);
    if ((int)t.size() > capacity) throw std::runtime_error("time_kernels: capacity too small");
    for (size_t i = 0; i < t.size(); ++i) ms[i] = t[i].second;
  })
}

tpuhip_ctx *tpuhip_module_ctx(tpuhip_module *m) { return m ? m->interp->context() : nullptr; }

}  // extern "C"

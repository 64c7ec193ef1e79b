// C ABI over the C++ ModuleInterpreter: exceptions become status codes.
#include <cstdarg>
#include <cstring>

#include "tpuhip/interpreter.hpp"
#include "tpuhip/mlir_text.hpp"
#include "tpuhip/tensor_file.hpp"

namespace tpuhip {
int set_error(int status, const char *fmt, ...);
MlirModule readMlirFile(const std::string &mlir_path);
}

struct tpuhip_npz {
  std::unique_ptr<tpuhip::TensorFile> file;
  std::vector<std::string> names;
};

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
    else if (k == "pair_convs")
      m->interp->pair_convs = value != 0;
    else if (k == "chain_convs")
      m->interp->chain_convs = value != 0;
    else if (k == "pack_inputs")
      m->interp->pack_inputs = value != 0;
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
    m->interp->setTensor(n, data, count, bidx);
  })
}

int tpuhip_module_set_tensor_i8(tpuhip_module *m, const char *name, const int8_t *data, size_t count,
                                int bidx) {
  GUARD(m, {
    if (!name || !data) throw std::runtime_error("set_tensor_i8: NULL argument");
    m->interp->setTensorI8(name, data, count, bidx);
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
  if (auto *f = dynamic_cast<FullyConnectedOpKernel *>(k)) return f->algo_name();
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

// ---- modules and tensors in files --------------------------------------------

int tpuhip_module_load_mlir(tpuhip_module *m, const char *mlir_path, const char *target_op) {
  GUARD(m, {
    if (!mlir_path) throw std::runtime_error("load_mlir: NULL path");
    m->interp->loadModuleFile(mlir_path, target_op ? target_op : "");
    m->tensor_names = m->interp->getAllTensorName();
  })
}

const char *tpuhip_module_weight_file(tpuhip_module *m) {
  return m ? m->interp->weightFilePath().c_str() : nullptr;
}

int tpuhip_module_num_ops(tpuhip_module *m) { return m ? (int)m->interp->opInfo().size() : 0; }

int tpuhip_module_op_info(tpuhip_module *m, int i, const char **name, const char **type, const char **quant) {
  GUARD(m, {
    auto &info = m->interp->opInfo();
    if (i < 0 || i >= (int)info.size()) throw std::runtime_error("op_info: index out of range");
    if (name) *name = info[i].name.c_str();
    if (type) *type = info[i].type.c_str();
    if (quant) *quant = info[i].quant.c_str();
  })
}

int tpuhip_module_interpret_files(tpuhip_module *m, const char *mlir_path, const char *tensor_in,
                                  const char *tensor_out, const char *dump_all_tensor) {
  GUARD(m, {
    if (!mlir_path || !tensor_in) throw std::runtime_error("interpret_files: NULL path");
    interpretFiles(*m->interp, mlir_path, tensor_in, tensor_out ? tensor_out : "",
                   dump_all_tensor ? dump_all_tensor : "");
    m->tensor_names = m->interp->getAllTensorName();
  })
}

int tpuhip_mlir_describe(const char *mlir_path, char *buf, size_t capacity, size_t *needed) {
  try {
    if (!mlir_path) throw std::runtime_error("mlir_describe: NULL path");
    const std::string text = describeModule(readMlirFile(mlir_path));
    if (needed) *needed = text.size() + 1;
    if (buf && capacity) {
      const size_t n = text.size() < capacity - 1 ? text.size() : capacity - 1;
      std::memcpy(buf, text.data(), n);
      buf[n] = '\0';
    }
  } catch (const std::exception &e) {
    return set_error(TPUHIP_ERR_INVALID, "%s", e.what());
  }
  return TPUHIP_OK;
}

int tpuhip_npz_open(const char *filename, int mode, tpuhip_npz **out) {
  if (!filename || !out) return set_error(TPUHIP_ERR_INVALID, "tpuhip_npz_open: NULL argument");
  try {
    auto *f = new tpuhip_npz();
    // 0: read only (must exist), 1: new empty file, 2: read what exists and allow changes
    f->file.reset(new TensorFile(filename, mode == 0, mode == 1));
    f->names = f->file->names();
    *out = f;
  } catch (const std::exception &e) {
    return set_error(TPUHIP_ERR_INVALID, "%s", e.what());
  }
  return TPUHIP_OK;
}

int tpuhip_npz_close(tpuhip_npz *f) {
  delete f;
  return TPUHIP_OK;
}

int tpuhip_npz_count(tpuhip_npz *f) { return f ? (int)f->names.size() : 0; }

const char *tpuhip_npz_name(tpuhip_npz *f, int i) {
  return f && i >= 0 && i < (int)f->names.size() ? f->names[i].c_str() : nullptr;
}

int tpuhip_npz_info(tpuhip_npz *f, const char *name, int64_t *dims8, int *ndim, char *kind, int *word_size) {
  GUARD(f, {
    auto *a = f->file->find(name ? name : "");
    if (!a) throw std::runtime_error(std::string("failed to find tensor ") + (name ? name : "(null)"));
    if (a->shape.size() > 8) throw std::runtime_error("npz_info: more than 8 dimensions");
    if (ndim) *ndim = (int)a->shape.size();
    if (dims8) for (size_t i = 0; i < a->shape.size(); ++i) dims8[i] = a->shape[i];
    if (kind) *kind = a->kind;
    if (word_size) *word_size = a->word_size;
  })
}

int tpuhip_npz_read_f32(tpuhip_npz *f, const char *name, float *dst, size_t count) {
  GUARD(f, {
    if (!name || (!dst && count)) throw std::runtime_error("npz_read_f32: NULL argument");
    if (!f->file->readTensor(name, dst, count)) {
      if (!f->file->find(name)) throw std::runtime_error(std::string("failed to find tensor ") + name + " to read");
      throw std::runtime_error(std::string("size does not match for tensor ") + name);
    }
  })
}

int tpuhip_npz_add_f32(tpuhip_npz *f, const char *name, const float *data, const int64_t *dims, int ndim) {
  GUARD(f, {
    if (!name || !dims || ndim < 0) throw std::runtime_error("npz_add_f32: bad argument");
    std::vector<int64_t> shape(dims, dims + ndim);
    if (!f->file->addTensor(name, data, shape))
      throw std::runtime_error(std::string("failed to add tensor ") + name + ", already exist");
    f->names = f->file->names();
  })
}

int tpuhip_npz_delete(tpuhip_npz *f, const char *name) {
  GUARD(f, {
    if (!f->file->deleteTensor(name ? name : ""))
      throw std::runtime_error(std::string("failed to find tensor ") + (name ? name : "(null)") + " to delete");
    f->names = f->file->names();
  })
}

int tpuhip_npz_keep(tpuhip_npz *f) { GUARD(f, f->file->keep()) }

}  // extern "C"

// ModuleInterpreter: builds the kernel list from a module description and runs
// it in program order on the context's stream.  Mirrors
// lib/Dialect/TPU/Interpreter/MlirModuleInterpreter.cpp:73-457.
#include "tpuhip/interpreter.hpp"

#include <algorithm>

#include <cstdio>
#include <cstdlib>

namespace tpuhip {

namespace {
[[noreturn]] void fail(const std::string &msg) { throw std::runtime_error(msg); }
void ck(int status, const char *what) {
  if (status != 0) fail(std::string(what) + ": " + tpuhip_last_error());
}

bool is_lut_op(const std::string &t) {
  static const char *names[] = {"tpu.sigmoid", "tpu.exp", "tpu.mish", "tpu.swish", "tpu.elu",
                                "tpu.softplus", "tpu.pow", "tpu.tanh", "tpu.log", "tpu.sqrt",
                                "tpu.lut"};
  for (auto n : names)
    if (t == n) return true;
  return false;
}
}  // namespace

ModuleInterpreter::ModuleInterpreter(int32_t batch, int device) {
  if (batch < 1) fail("ModuleInterpreter: batch < 1");
  CPUOpKernel::max_batch_size = batch;
  ck(tpuhip_ctx_create(device, &ctx_), "ModuleInterpreter");
  valueMapping.ctx = ctx_;
}

ModuleInterpreter::~ModuleInterpreter() {
  if (ctx_) tpuhip_sync(ctx_);
  kernel_list_.clear();
  kernel_map_.clear();
  activationMapping.clear();
  valueMapping.clear();
  if (ctx_) tpuhip_ctx_destroy(ctx_);
}

void ModuleInterpreter::updateWeightMap(const std::string &name, const float *data, size_t count) {
  auto w = std::make_shared<WeightData>();
  w->data.assign(data, data + count);
  weightMapping[name] = w;
}

void ModuleInterpreter::loadModule(ModuleDesc &module, std::string target_op) {
  updateKernelList(module, target_op);
  fuseKernels();
  chainConvs();
  pairConvs();
  packInputs();
  spreadDirtiness();
}

// The dirty flag of the reference (MlirModuleInterpreter.cpp:85-116, 383-405) belongs to one
// kernel; here several kernels can share one launch.  After a partial reload a rebuilt (dirty)
// add, table op or second conv of a pair may have been folded into a retained (clean) conv
// whose launch is the only thing that writes its fresh result tensor -- so within a launch
// group one dirty member makes every member dirty.
void ModuleInterpreter::spreadDirtiness() {
  for (bool changed = true; changed;) {   // groups chain through a shared conv: to a fixed point
    changed = false;
    for (auto &group : launch_groups_) {
      bool any = false, all = true;
      for (auto *k : group) {
        any = any || k->dirty;
        all = all && k->dirty;
      }
      if (any && !all) {
        for (auto *k : group) k->dirty = true;
        changed = true;
      }
    }
  }
}

// Work that rides in a dense conv's epilogue instead of running as a kernel of its own
// (same bytes, fewer launches and fewer passes over the tensors):
//  * a table op (Lut / LeakyRelu / Clip) whose input is the conv result;
//  * a two-input EltwiseAdd whose later-produced input is the conv's final result
//    (after the fused table, if any).
// Recomputed from scratch on every load so that rebuilt kernels never keep stale links.
void ModuleInterpreter::fuseKernels() {
  std::map<TensorData *, std::pair<int, Conv2DOpKernel *>> producer;   // final result -> (position, conv)
  std::map<TensorData *, int> position;                               // tensor -> producing position
  std::vector<Conv2DOpKernel *> fused_convs;
  int pos = 0;
  launch_groups_.clear();
  for (auto &k : kernel_list_) {
    if (auto *c = dynamic_cast<Conv2DOpKernel *>(k.get())) c->clear_fusion();
    if (auto *e = dynamic_cast<EltwiseAddOpKernel *>(k.get())) e->fused_into_producer = false;
    if (auto *l = dynamic_cast<LutOpKernel *>(k.get())) l->fused_into_producer = false;
    if (auto *q = dynamic_cast<PoolingOpKernel *>(k.get())) q->fused_into_producer = false;
  }
  const char *env = getenv("TPUHIP_FUSE");
  if (!fuse_eltwise || (env && atoi(env) == 0)) return;
  for (auto &k : kernel_list_) {
    ++pos;
    if (auto *c = dynamic_cast<Conv2DOpKernel *>(k.get())) {
      producer[c->result().get()] = {pos, c};
      position[c->result().get()] = pos;
      continue;
    }
    if (auto *l = dynamic_cast<LutOpKernel *>(k.get())) {
      position[l->result().get()] = pos;
      auto it = producer.find(l->input().get());
      if (it == producer.end() || !it->second.second->can_fuse_lut()) continue;
      Conv2DOpKernel *conv = it->second.second;
      if (conv->result().get() != l->input().get()) continue;
      const int conv_pos = it->second.first;
      conv->fuse_lut(l->table, l->result());
      l->fused_into_producer = true;
      launch_groups_.push_back({conv, l});
      producer.erase(it);
      producer[l->result().get()] = {conv_pos, conv};   // an add may follow the table
      fused_convs.push_back(conv);
      continue;
    }
    if (auto *q = dynamic_cast<PoolingOpKernel *>(k.get())) {
      // a max pool straight behind the stem conv runs in the conv's launch
      position[q->result().get()] = pos;
      auto it = producer.find(q->input().get());
      if (!q->is_max() || it == producer.end()) continue;
      Conv2DOpKernel *conv = it->second.second;
      if (conv->result().get() != q->input().get() || !conv->can_fuse_pool(q->pool_desc())) continue;
      conv->fuse_pool(q->pool_desc(), q->result());
      q->fused_into_producer = true;
      launch_groups_.push_back({conv, q});
      producer.erase(it);
      fused_convs.push_back(conv);
      continue;
    }
    auto *e = dynamic_cast<EltwiseAddOpKernel *>(k.get());
    if (!e) {
      auto it = activationMapping.find(k->name);
      if (it != activationMapping.end()) position[it->second.get()] = pos;
      continue;
    }
    position[e->result().get()] = pos;
    if (e->inputs().size() != 2) continue;
    // the conv must be the later of the two producers
    int conv_idx = -1, best_pos = -1;
    for (int i = 0; i < 2; ++i) {
      auto it = producer.find(e->inputs()[i].get());
      if (it != producer.end() && it->second.first > best_pos && it->second.second->can_fuse_add()) {
        best_pos = it->second.first;
        conv_idx = i;
      }
    }
    if (conv_idx < 0) continue;
    TensorData *other = e->inputs()[1 - conv_idx].get();
    auto po = position.find(other);
    if (po == position.end() || po->second >= best_pos) continue;   // other operand not ready yet
    Conv2DOpKernel *conv = producer[e->inputs()[conv_idx].get()].second;
    if (e->inputs()[0].get() == e->inputs()[1].get()) continue;
    conv->fuse_add(e->inputs()[1 - conv_idx], e->result(), e->multipliers()[1 - conv_idx],
                   e->multipliers()[conv_idx], e->rshift_value(), e->relu());
    e->fused_into_producer = true;
    launch_groups_.push_back({conv, e});   // (conv, table) and (conv, add) chain through the conv
    producer.erase(e->inputs()[conv_idx].get());   // one add per conv
    if (std::find(fused_convs.begin(), fused_convs.end(), conv) == fused_convs.end())
      fused_convs.push_back(conv);
  }
  if (keep_all_tensors) return;
  // outputs only: an intermediate of a fused chain that nothing else reads, and that is
  // not a module output, need not be written
  std::map<TensorData *, int> readers;
  std::map<TensorData *, std::string> tensor_name;
  for (auto &k : kernel_list_)
    for (auto &opd : k->operands())
      if (opd.act) ++readers[opd.act.get()];
  for (auto &kv : activationMapping) tensor_name[kv.second.get()] = kv.first;
  auto droppable = [&](TensorData *t) {
    const bool is_output = std::find(output_details.begin(), output_details.end(),
                                     tensor_name[t]) != output_details.end();
    return !is_output && readers[t] == 1;
  };
  for (Conv2DOpKernel *conv : fused_convs) {
    // the one reader of the conv result is the fused table op or the fused add
    if (droppable(conv->result().get())) conv->set_store_result(false);
    if (conv->has_fused_lut() && conv->final_result().get() != conv->result().get() &&
        conv->has_fused_add() && droppable(conv->final_result().get()))
      conv->set_store_lut(false);
  }
}

// A pointwise conv -- with the add folded into it, if any -- and the pointwise conv that reads its
// final result become one launch where the library covers the pair (the 1x1 expansion + add that
// closes a bottleneck block and the 1x1 reduction that opens the next): the second conv's work
// moves to the position of the first, which is legal because its only activation operand is
// produced there and nothing reads its result before its own position.  The intermediate tensor
// is still written (other kernels read it).  Runs after the add / table fusions.
void ModuleInterpreter::chainConvs() {
  const char *env = getenv("TPUHIP_CHAIN");
  if (!chain_convs || (env && atoi(env) == 0)) return;
  std::vector<Conv2DOpKernel *> convs;
  for (auto &k : kernel_list_)
    if (auto *c = dynamic_cast<Conv2DOpKernel *>(k.get())) convs.push_back(c);
  for (size_t i = 0; i < convs.size(); ++i)
    for (size_t j = i + 1; j < convs.size(); ++j)
      if (convs[i]->chain_with(*convs[j])) {
        launch_groups_.push_back({convs[i], convs[j]});
        break;
      }
}

// Convs that read the same tensor through the same window geometry (the projection shortcut
// and the first 1x1 of a residual block, for one) become one launch: the second one's work
// moves to the position of the first, which is legal because its only activation operand
// is available there and nothing reads its result before its own position.  Runs after the
// add / table fusions, which take precedence.
void ModuleInterpreter::pairConvs() {
  std::vector<Conv2DOpKernel *> convs;
  for (auto &k : kernel_list_)
    if (auto *c = dynamic_cast<Conv2DOpKernel *>(k.get())) convs.push_back(c);
  const char *env = getenv("TPUHIP_PAIR");
  if (pair_convs && !(env && atoi(env) == 0)) {
    for (size_t i = 0; i < convs.size(); ++i)
      for (size_t j = i + 1; j < convs.size(); ++j)
        if (convs[i]->can_pair_with(*convs[j])) {
          try {
            convs[i]->pair_with(*convs[j]);
            launch_groups_.push_back({convs[i], convs[j]});
          } catch (const std::exception &) {
            // shapes the packed form does not cover stay two launches
          }
          break;
        }
  }
  // paired kernels keep their host operands so that a reload can pair them again
  for (auto *c : convs)
    if (!c->is_paired_first() && !c->is_paired_second() && !c->is_chain_first() && !c->is_chain_second())
      c->release_host_weights();
}

// A graph input of at most 4 channels whose only readers are convs on the stem path -- they take a
// pixel as one dword -- is laid out at a channel stride of 4 instead of 16: a quarter of the bytes
// to write at set_tensor and to fetch in the stem.  Decided anew at every load (a reload can change
// the readers), after pairing, which can take a stem conv off the stem path.
void ModuleInterpreter::packInputs() {
  const char *env = getenv("TPUHIP_PACK_INPUT");
  const bool on = pack_inputs && !(env && atoi(env) == 0);
  for (auto &k : kernel_list_) {
    if (!dynamic_cast<InputOpKernel *>(k.get())) continue;
    auto it = activationMapping.find(k->name);
    if (it == activationMapping.end()) continue;
    TensorData *t = it->second.get();
    if (t->f32 || t->is_unsigned || t->c > 4) continue;
    std::vector<Conv2DOpKernel *> convs;   // convs whose activation input is t
    bool all = on;
    for (auto &r : kernel_list_) {
      if (r.get() == k.get()) continue;
      bool reads = false;
      for (auto &opd : r->operands())
        if (opd.act && opd.act.get() == t) reads = true;
      if (!reads) continue;
      auto *c = dynamic_cast<Conv2DOpKernel *>(r.get());
      if (c && c->input().get() == t) convs.push_back(c);
      if (!c || c->input().get() != t || !c->reads_dword_pixels()) all = false;
    }
    int want = (all && !convs.empty()) ? 4 : tpuhip_channel_stride(t->c);
    if (want == 4)
      for (auto *c : convs)
        if (!c->set_input_stride(4)) want = tpuhip_channel_stride(t->c);
    if (want != 4)
      for (auto *c : convs) c->set_input_stride(want);
    t->set_channel_stride(want);
  }
}

// MlirModuleInterpreter.cpp:85-116
bool ModuleInterpreter::isKernelDirty(std::shared_ptr<CPUOpKernel> &krnl, OpDesc *op) {
  if (op->type == "tpu.input") return false;
  if (krnl->dirty) return true;
  auto new_signature = CPUOpKernel::generateSignature(*op);
  bool dirty = krnl->signature != new_signature;
  if (!dirty) {
    for (auto &opd : op->operands) {
      if (opd.empty()) continue;
      auto it = kernel_map_.find(opd);
      if (it == kernel_map_.end()) continue;
      if (it->second && it->second->dirty) {
        dirty = true;
        break;
      }
    }
  }
  return dirty;
}

// MlirModuleInterpreter.cpp:118-350
void ModuleInterpreter::updateKernelList(ModuleDesc &module, std::string &target_op) {
  kernel_list_.clear();
  static_cast<std::map<std::string, SyncedData> &>(valueMapping).clear();
  output_details = module.returns;
  bool completed = false;
  for (auto &opd : module.ops) {
    if (completed) break;
    OpDesc *op = &opd;
    const std::string &name = op->name;
    if (!target_op.empty() && target_op == name) completed = true;

    auto it = kernel_map_.find(name);
    if (it != kernel_map_.end() && it->second && op->type != "tpu.reshape") {
      auto &krnl = it->second;
      bool dirty = isKernelDirty(krnl, op);
      if (!dirty) {
        krnl->dirty = false;
        krnl->op = op;
        valueMapping[name] = activationMapping[name];
        valueMapping.shapes[name] = op->shape;
        kernel_list_.emplace_back(krnl);
        continue;
      }
      activationMapping.erase(name);
    }

    std::shared_ptr<CPUOpKernel> krnl;
    const std::string &t = op->type;
    if (t == "tpu.input") {
      // a reloaded module keeps its input kernel (and the data set on it)
      krnl = std::make_shared<InputOpKernel>(*op, valueMapping, weightMapping, input_details);
    } else if (t == "tpu.conv_2d") {
      krnl = std::make_shared<Conv2DOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.deconv_2d") {
      krnl = std::make_shared<DeConv2DOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.fully_connected") {
      krnl = std::make_shared<FullyConnectedOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.eltwise_add") {
      krnl = std::make_shared<EltwiseAddOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.eltwise_max") {
      krnl = std::make_shared<EltwiseMaxOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.eltwise_min") {
      krnl = std::make_shared<EltwiseMinOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.eltwise_mul") {
      krnl = std::make_shared<EltwiseMulOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.broadcast_add") {
      krnl = std::make_shared<BroadcastAddOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.broadcast_mul") {
      krnl = std::make_shared<BroadcastMulOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.broadcast_sub") {
      krnl = std::make_shared<BroadcastSubOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.pool_avg_2d" || t == "tpu.pool_max_2d") {
      krnl = std::make_shared<PoolingOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.leaky_relu") {
      krnl = std::make_shared<LeakyReluOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.pad") {
      krnl = std::make_shared<PadOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.crop") {
      krnl = std::make_shared<CropOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.permute") {
      krnl = std::make_shared<PermuteOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.reorg") {
      krnl = std::make_shared<ReorgOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.tile") {
      krnl = std::make_shared<TileOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.reverse") {
      krnl = std::make_shared<ReverseOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.dilate") {
      krnl = std::make_shared<DilateOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.reflection_pad") {
      krnl = std::make_shared<ReflectionPadOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.shuffle_channel") {
      krnl = std::make_shared<ShuffleChannelOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.pixelshuffle") {
      krnl = std::make_shared<DepthToSpaceOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.quant") {
      krnl = std::make_shared<QuantOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.scale_lut") {
      krnl = std::make_shared<ScaleLutOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.prelu") {
      krnl = std::make_shared<PReluOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.clip") {
      krnl = std::make_shared<ClipOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.reduce_mean" || t == "tpu.reduce_sum" || t == "tpu.reduce_max" || t == "tpu.reduce_min") {
      krnl = std::make_shared<ReduceOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.lrn") {
      krnl = std::make_shared<LrnOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.zero_mask") {
      krnl = std::make_shared<ZeroMaskOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.mul_const") {
      krnl = std::make_shared<MulConstOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.swap_channel") {
      krnl = std::make_shared<SwapChannelOpKernel>(*op, valueMapping, weightMapping);
    } else if (is_lut_op(t)) {
      krnl = std::make_shared<LutOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.relu") {
      krnl = std::make_shared<ReluOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.upsample") {
      krnl = std::make_shared<UpsampleOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.concat") {
      krnl = std::make_shared<ConcatOpKernel>(*op, valueMapping, weightMapping);
    } else if (t == "tpu.reshape") {
      if (op->operands.empty()) fail("reshape '" + name + "': no operand");
      const std::string &src = op->operands[0];
      auto vit = valueMapping.find(src);
      if (vit == valueMapping.end()) fail("reshape '" + name + "': operand '" + src + "' not found");
      if (ReshapeOpKernel::is_alias(valueMapping.shapes[src], op->shape)) {
        // zero-copy alias (MlirModuleInterpreter.cpp:331-338)
        auto resTensor = vit->second;
        activationMapping[name] = resTensor;
        valueMapping[name] = resTensor;
        valueMapping.shapes[name] = op->shape;
        kernel_map_[name] = kernel_map_[src];
        continue;
      }
      krnl = std::make_shared<ReshapeOpKernel>(*op, valueMapping, weightMapping);
    } else {
      fail("no support " + t + " op in interpreter_v2");
    }
    activationMapping[name] = valueMapping[name];
    kernel_map_[name] = krnl;
    kernel_list_.emplace_back(krnl);
  }
}

// MlirModuleInterpreter.cpp:371-381
void ModuleInterpreter::invokeTo(std::string name, int32_t bidx) {
  for (auto &kv : valueMapping) kv.second->set_batch_idx(bidx);
  for (auto &krnl : kernel_list_) {
    krnl->invoke();
    if (!name.empty() && name == krnl->name) break;
  }
}

// MlirModuleInterpreter.cpp:383-405
void ModuleInterpreter::fastInvokeAllBatch(std::string name, int32_t batch) {
  bool last_batch = false;
  for (int i = 0; i < batch; i++) {
    if (i == batch - 1) last_batch = true;
    for (auto &kv : valueMapping) kv.second->set_batch_idx(i);
    for (auto &krnl : kernel_list_) {
      if (krnl->dirty) {
        krnl->invoke();
        if (last_batch) krnl->dirty = false;
      }
      if (!name.empty() && name == krnl->name) break;
    }
  }
}

void ModuleInterpreter::setTensor(std::string &name, const std::vector<float> &data, int32_t bidx) {
  setTensor(name, data.data(), data.size(), bidx);
}

void ModuleInterpreter::setTensor(std::string &name, const float *data, size_t count, int32_t bidx) {
  auto it = activationMapping.find(name);
  if (it == activationMapping.end()) fail(" Not Find Op name: " + name + " tensor");
  it->second->assign(data, count, bidx);
}

void ModuleInterpreter::setTensorI8(const std::string &name, const int8_t *data, size_t count, int32_t bidx) {
  auto it = activationMapping.find(name);
  if (it == activationMapping.end()) fail(" Not Find Op name: " + name + " tensor");
  it->second->assign_i8(data, count, bidx);
}

std::shared_ptr<std::vector<float>> ModuleInterpreter::getTensor(std::string &name, int32_t bidx) {
  auto it = activationMapping.find(name);
  if (it == activationMapping.end()) fail(" Not Find Op name: " + name + " tensor");
  return it->second->tensor(bidx);
}

void ModuleInterpreter::getTensorI8(const std::string &name, int8_t *dst, size_t num, int32_t bidx) {
  auto it = activationMapping.find(name);
  if (it == activationMapping.end()) fail(" Not Find Op name: " + name + " tensor");
  it->second->read_i8(dst, num, bidx);
}

std::vector<int64_t> ModuleInterpreter::getTensorShape(std::string &name) {
  auto it = valueMapping.shapes.find(name);
  if (it == valueMapping.shapes.end()) fail(" Not Find Op name: " + name + " tensor");
  return it->second;
}

std::string ModuleInterpreter::getDataType(std::string &name) {
  auto it = kernel_map_.find(name);
  if (it == kernel_map_.end() || !it->second) fail(" Not Find Op name: " + name + " tensor");
  return it->second->get_data_type();
}

void ModuleInterpreter::dump(std::string &name) {
  for (auto &krnl : kernel_list_)
    if (krnl->get_name() == name) return krnl->dump();
  fprintf(stderr, " Not Find Op name: %s tensor \n", name.c_str());
}

std::vector<std::string> ModuleInterpreter::getAllTensorName() {
  std::vector<std::string> ret;
  for (auto &kv : activationMapping) ret.push_back(kv.first);
  return ret;
}

void ModuleInterpreter::sync() { ck(tpuhip_sync(ctx_), "sync"); }

std::vector<std::pair<std::string, float>> ModuleInterpreter::timeKernels(int32_t bidx, int iters) {
  // Every kernel of a normal invoke carries its own pair of HIP events, which the
  // dispatch fills with the begin and end of its execution on the module's stream:
  // the duration of the kernel itself, in place, with the caches as a real step
  // leaves them.  An op that launches no kernel reports 0.
  if (iters < 1) iters = 1;
  for (auto &kv : valueMapping) kv.second->set_batch_idx(bidx);
  const size_t nk = kernel_list_.size();
  std::vector<void *> e0(nk, nullptr), e1(nk, nullptr);
  for (size_t i = 0; i < nk; ++i) {
    ck(tpuhip_event_create(ctx_, &e0[i]), "timeKernels");
    ck(tpuhip_event_create(ctx_, &e1[i]), "timeKernels");
  }
  std::vector<double> acc(nk, 0.0);
  for (int it = 0; it < iters; ++it) {
    size_t i = 0;
    std::vector<bool> launched(nk, false);
    for (auto &krnl : kernel_list_) {
      auto *el = dynamic_cast<EltwiseAddOpKernel *>(krnl.get());
      auto *lu = dynamic_cast<LutOpKernel *>(krnl.get());
      auto *cv = dynamic_cast<Conv2DOpKernel *>(krnl.get());
      auto *po = dynamic_cast<PoolingOpKernel *>(krnl.get());
      const bool runs = !(dynamic_cast<InputOpKernel *>(krnl.get()) || (cv && (cv->is_paired_second() || cv->is_chain_second())) ||
                          (el && el->fused_into_producer) || (lu && lu->fused_into_producer) ||
                          (po && po->fused_into_producer));
      if (runs) ck(tpuhip_ctx_set_kernel_events(ctx_, e0[i], e1[i]), "timeKernels");
      krnl->invoke();
      launched[i] = runs;
      ++i;
    }
    ck(tpuhip_ctx_set_kernel_events(ctx_, nullptr, nullptr), "timeKernels");
    ck(tpuhip_sync(ctx_), "timeKernels");
    for (i = 0; i < nk; ++i) {
      if (!launched[i]) continue;
      float ms = 0;
      ck(tpuhip_event_elapsed_ms(ctx_, e0[i], e1[i], &ms), "timeKernels");
      acc[i] += ms;
    }
  }
  std::vector<std::pair<std::string, float>> out;
  size_t i = 0;
  for (auto &krnl : kernel_list_) out.emplace_back(krnl->name, (float)(acc[i++] / iters));
  for (size_t k = 0; k < nk; ++k) {
    tpuhip_event_destroy(ctx_, e0[k]);
    tpuhip_event_destroy(ctx_, e1[k]);
  }
  return out;
}

}  // namespace tpuhip

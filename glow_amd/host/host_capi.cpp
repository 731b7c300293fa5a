// Flat C wrappers over the C++ host layer (declared in glow_mi355x_host.h).
#include "DeviceManager.h"

#include "glow_mi355x_host.h"

#include <future>

using namespace glow_mi355x;

struct mi355x_host_module {
  Module module;
  std::map<int, std::unique_ptr<MI355XFunction>> compiled;
  explicit mi355x_host_module(const char *n) : module(n ? n : "module") {}
};

struct mi355x_host_dm {
  MI355XDeviceManager dm;
  std::map<std::string, const Module *> owners;
  explicit mi355x_host_dm(const DeviceConfig &c) : dm(c) {}
};

namespace {
thread_local std::string g_msg;

int fail(const Error &e) {
  g_msg = e.message();
  return -(int)e.code();
}
int failMsg(ErrorCode c, const std::string &m) {
  g_msg = m;
  return -(int)c;
}
Type makeType(int kind, const int64_t *dims, int nd, float scale, int32_t offset) {
  return Type((ElemKind)kind, std::vector<int64_t>(dims, dims + (nd > 0 ? nd : 0)), scale, offset);
}
bool kindOk(int k) { return k >= 0 && k <= (int)ElemKind::Int16QTy; }
Function *fn(mi355x_host_module *m, int f) {
  if (!m || f < 0 || (size_t)f >= m->module.functions().size()) return nullptr;
  return m->module.functions()[(size_t)f].get();
}
} // namespace

extern "C" {

const char *mi355x_host_last_error(void) { return g_msg.c_str(); }
const char *mi355x_host_error_name(int code) { return errorCodeName((ErrorCode)(code < 0 ? -code : code)); }

mi355x_host_module *mi355x_host_module_create(const char *name) { return new mi355x_host_module(name); }
void mi355x_host_module_destroy(mi355x_host_module *m) { delete m; }

int mi355x_host_add_constant(mi355x_host_module *m, const char *name, int kind, const int64_t *dims,
                             int nd, float scale, int32_t offset, const void *payload) {
  if (!m || !name || !kindOk(kind) || (nd > 0 && !dims))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid constant description");
  return m->module.createConstant(name, makeType(kind, dims, nd, scale, offset), payload);
}

int mi355x_host_add_placeholder(mi355x_host_module *m, const char *name, int kind,
                                const int64_t *dims, int nd, float scale, int32_t offset) {
  if (!m || !name || !kindOk(kind) || (nd > 0 && !dims))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid placeholder description");
  return m->module.createPlaceholder(name, makeType(kind, dims, nd, scale, offset));
}

int mi355x_host_create_function(mi355x_host_module *m, const char *name) {
  if (!m || !name) return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid function name");
  return m->module.createFunction(name)->index();
}

int mi355x_host_add_activation(mi355x_host_module *m, int function, const char *name, int kind,
                               const int64_t *dims, int nd, float scale, int32_t offset) {
  Function *f = fn(m, function);
  if (!f || !name || !kindOk(kind) || (nd > 0 && !dims))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid activation description");
  return f->createActivation(name, makeType(kind, dims, nd, scale, offset));
}

int mi355x_host_add_view(mi355x_host_module *m, const char *name, int source, int kind,
                         const int64_t *dims, int nd, float scale, int32_t offset) {
  if (!m || !name || !kindOk(kind) || (nd > 0 && !dims))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid view description");
  const int id = m->module.createView(name, source, makeType(kind, dims, nd, scale, offset));
  if (id < 0)
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED,
                   "view " + std::string(name) + " does not fit its source");
  return id;
}

int mi355x_host_add_view_at(mi355x_host_module *m, const char *name, int source, int kind,
                            const int64_t *dims, int nd, float scale, int32_t offset,
                            size_t byte_offset) {
  if (!m || !name || !kindOk(kind) || (nd > 0 && !dims))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid view description");
  const int id =
      m->module.createView(name, source, makeType(kind, dims, nd, scale, offset), byte_offset);
  if (id < 0)
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED,
                   "view " + std::string(name) +
                       " does not fit its source (or slices an activation)");
  return id;
}

int mi355x_host_add_instruction(mi355x_host_module *m, int function, int kind, const char *name,
                                const int *operands, int n_operands, const int64_t *iattrs,
                                int n_iattrs, const float *fattrs, int n_fattrs) {
  Function *f = fn(m, function);
  if (!f || n_operands < 0 || n_iattrs < 0 || n_fattrs < 0)
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "invalid instruction description");
  return f->addInstruction((Kind)kind, name ? name : "",
                           std::vector<int>(operands, operands + n_operands),
                           std::vector<int64_t>(iattrs, iattrs + n_iattrs),
                           std::vector<float>(fattrs, fattrs + n_fattrs));
}

int mi355x_host_is_op_supported(mi355x_host_module *m, int kind, const int *operands, int n_operands,
                                const int64_t *iattrs, int n_iattrs, const float *fattrs,
                                int n_fattrs) {
  if (!m) return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "module is NULL");
  Instruction I;
  I.kind = (Kind)kind;
  I.name = "probe";
  I.operands.assign(operands, operands + n_operands);
  I.iattrs.assign(iattrs, iattrs + n_iattrs);
  I.fattrs.assign(fattrs, fattrs + n_fattrs);
  std::string why;
  const bool ok = MI355XBackend().isOpSupported(m->module, I, &why);
  if (!ok) g_msg = why;
  return ok ? 1 : 0;
}

int mi355x_host_compile(mi355x_host_module *m, int function, int options) {
  Function *f = fn(m, function);
  if (!f) return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "no such function");
  BackendOptions o;
  o.precomputeWeightRowSums = (options & MI355X_HOST_OPT_WEIGHT_ROW_SUMS) != 0;
  o.fuseAddRelu = (options & MI355X_HOST_OPT_FUSE_ADD_RELU) != 0;
  o.fuseConvAdd = (options & MI355X_HOST_OPT_FUSE_CONV_ADD) != 0;
  o.spaceToDepthStem = (options & MI355X_HOST_OPT_SPACE_TO_DEPTH_STEM) != 0;
  o.fuseSlsChains = (options & MI355X_HOST_OPT_FUSE_SLS_CHAINS) != 0;
  o.fuseTransposeMatMul = (options & MI355X_HOST_OPT_FUSE_TRANSPOSE_MATMUL) != 0;
  o.fuseFcRelu = (options & MI355X_HOST_OPT_FUSE_FC_RELU) != 0;
  o.padTableRows = (options & MI355X_HOST_OPT_PAD_TABLE_ROWS) != 0;
  o.fuseInsert = (options & MI355X_HOST_OPT_FUSE_INSERT) != 0;
  o.fuseDequantizeSigmoid = (options & MI355X_HOST_OPT_FUSE_DEQUANTIZE_SIGMOID) != 0;
  o.deriveBagOffsets = (options & MI355X_HOST_OPT_DERIVE_BAG_OFFSETS) != 0;
  o.reuseActivations = (options & MI355X_HOST_OPT_REUSE_ACTIVATIONS) != 0;
  o.fuseQuantizeStem = (options & MI355X_HOST_OPT_FUSE_QUANTIZE_STEM) != 0;
  o.splitK = (options & MI355X_HOST_OPT_SPLIT_K) != 0;
  auto r = MI355XBackend().compile(*f, o);
  if (!r) return fail(r.error());
  m->compiled[function] = std::move(r.get());
  return 0;
}

int mi355x_host_describe(mi355x_host_module *m, int function, char *buf, size_t cap) {
  if (!m || !m->compiled.count(function))
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "function is not compiled");
  const std::string s = m->compiled[function]->describe();
  if (buf && cap) {
    const size_t n = std::min(cap - 1, s.size());
    std::memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return (int)s.size() + 1;
}

int mi355x_host_bundle_sizes(mi355x_host_module *m, int function, uint64_t out[4]) {
  if (!m || !m->compiled.count(function) || !out)
    return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "function is not compiled");
  const RuntimeBundle &rb = m->compiled[function]->getRuntimeBundle();
  out[0] = rb.constantWeightVarsMemSize;
  out[1] = rb.generatedConstantsMemSize;
  out[2] = rb.mutableWeightVarsMemSize;
  out[3] = rb.activationsMemSize;
  return 0;
}

static DeviceConfig makeConfig(int device, uint64_t memory_bytes, int graphs) {
  DeviceConfig c;
  c.deviceID = device;
  c.deviceMemory = memory_bytes;
  c.useLaunchGraphs = graphs != 0;
  if (graphs > 1) c.graphBranches = graphs; // 1 keeps the default
  if (graphs < 0) {
    c.graphBranches = -graphs;
    c.autotuneBranches = false;
  }
  return c;
}

mi355x_host_dm *mi355x_host_dm_create(int device, uint64_t memory_bytes, int graphs) {
  return new mi355x_host_dm(makeConfig(device, memory_bytes, graphs));
}

mi355x_host_dm *mi355x_host_dm_create_opts(int device, uint64_t memory_bytes, int graphs,
                                           int slws_math) {
  DeviceConfig c = makeConfig(device, memory_bytes, graphs);
  c.slwsMath = slws_math;
  return new mi355x_host_dm(c);
}
void mi355x_host_dm_destroy(mi355x_host_dm *dm) { delete dm; }

int mi355x_host_dm_init(mi355x_host_dm *dm) {
  if (!dm) return failMsg(ErrorCode::RUNTIME_ERROR, "device manager is NULL");
  Error e = dm->dm.init();
  return e ? fail(e) : 0;
}
int mi355x_host_dm_stop(mi355x_host_dm *dm) {
  if (!dm) return failMsg(ErrorCode::RUNTIME_ERROR, "device manager is NULL");
  Error e = dm->dm.stop(true);
  return e ? fail(e) : 0;
}

int mi355x_host_dm_add_network(mi355x_host_dm *dm, mi355x_host_module *m) {
  if (!dm || !m) return failMsg(ErrorCode::RUNTIME_ERROR, "NULL handle");
  FunctionMapTy fm;
  for (auto &kv : m->compiled) fm[kv.second->name()] = kv.second.get();
  std::promise<Error> p;
  auto fut = p.get_future();
  dm->dm.addNetwork(&m->module, fm, [&p](const Module *, Error e) { p.set_value(std::move(e)); });
  Error e = fut.get();
  return e ? fail(e) : 0;
}

int mi355x_host_dm_add_functions(mi355x_host_dm *dm, mi355x_host_module *m, const int *functions,
                                 int n) {
  if (!dm || !m || n < 0 || (n > 0 && !functions))
    return failMsg(ErrorCode::RUNTIME_ERROR, "NULL handle");
  FunctionMapTy fm;
  for (int i = 0; i < n; i++) {
    auto it = m->compiled.find(functions[i]);
    if (it == m->compiled.end())
      return failMsg(ErrorCode::COMPILE_CONTEXT_MALFORMED, "function is not compiled");
    fm[it->second->name()] = it->second.get();
  }
  std::promise<Error> p;
  auto fut = p.get_future();
  dm->dm.addNetwork(&m->module, fm, [&p](const Module *, Error e) { p.set_value(std::move(e)); });
  Error e = fut.get();
  return e ? fail(e) : 0;
}

int mi355x_host_dm_transfer_static_placeholder(mi355x_host_dm *dm, mi355x_host_module *m,
                                               const char *name, void *buffer, size_t bytes) {
  if (!dm || !m || !name || (!buffer && bytes))
    return failMsg(ErrorCode::RUNTIME_ERROR, "NULL argument");
  Tensor t = Tensor::unowned(Type(ElemKind::Int8QTy, {(int64_t)bytes}), buffer, bytes);
  std::promise<Error> p;
  auto fut = p.get_future();
  dm->dm.transferStaticPlaceholderToDevice(&m->module, name, &t,
                                           [&p](Error e) { p.set_value(std::move(e)); });
  Error e = fut.get();
  return e ? fail(e) : 0;
}

int mi355x_host_dm_evict_network(mi355x_host_dm *dm, const char *name) {
  if (!dm || !name) return failMsg(ErrorCode::RUNTIME_ERROR, "NULL handle");
  std::promise<Error> p;
  auto fut = p.get_future();
  dm->dm.evictNetwork(name, [&p](std::string, Error e) { p.set_value(std::move(e)); });
  Error e = fut.get();
  return e ? fail(e) : 0;
}

int mi355x_host_dm_run(mi355x_host_dm *dm, const char *name, const char *const *names,
                       void *const *buffers, const size_t *bytes, int n) {
  if (!dm || !name || n < 0 || (n > 0 && (!names || !buffers || !bytes)))
    return failMsg(ErrorCode::RUNTIME_ERROR, "invalid run arguments");
  auto ctx = std::unique_ptr<ExecutionContext>(new ExecutionContext());
  std::vector<Tensor> tensors;
  tensors.reserve((size_t)n);
  for (int i = 0; i < n; i++) {
    tensors.push_back(Tensor::unowned(Type(ElemKind::Int8QTy, {(int64_t)bytes[i]}), buffers[i], bytes[i]));
    ctx->getPlaceholderBindings()->insert(names[i], &tensors.back());
  }
  std::promise<Error> p;
  auto fut = p.get_future();
  dm->dm.runFunction(name, std::move(ctx),
                     [&p](RunIdentifierTy, Error e, std::unique_ptr<ExecutionContext>) {
                       p.set_value(std::move(e));
                     });
  Error e = fut.get();
  return e ? fail(e) : 0;
}

int mi355x_host_dm_time_function(mi355x_host_dm *dm, const char *name, int iterations,
                                 float *ms_per_iteration) {
  if (!dm || !name || !ms_per_iteration) return failMsg(ErrorCode::RUNTIME_ERROR, "NULL argument");
  auto r = dm->dm.timeFunction(name, iterations);
  if (!r) return fail(r.error());
  *ms_per_iteration = r.get();
  return 0;
}

uint64_t mi355x_host_dm_maximum_memory(mi355x_host_dm *dm) { return dm ? dm->dm.getMaximumMemory() : 0; }
uint64_t mi355x_host_dm_available_memory(mi355x_host_dm *dm) { return dm ? dm->dm.getAvailableMemory() : 0; }

} // extern "C"

#include "DeviceManager.h"

#include "glow_mi355x.h"

#include <future>

namespace glow_mi355x {

namespace {
// The other half of MI355XFunction::derivedBagOffsets: `lengths` (n int32) has
// just been copied into placeholder `name`; the positions its lookups read go
// to the function's scratch. `staged` keeps the host vectors alive until the
// caller has synchronised the stream.
int uploadBagOffsets(const MI355XFunction &fn, const DeviceBindings &b, const std::string &name,
                     const void *lengths, size_t bytes, void *stream,
                     std::vector<std::vector<int32_t>> &staged) {
  for (const auto &d : fn.derivedBagOffsets) {
    if (d.lengths != name) continue;
    staged.push_back(MI355XFunction::bagOffsets(static_cast<const int32_t *>(lengths),
                                                bytes / sizeof(int32_t), d.segments));
    const int rc = mi355x_memcpy_h2d(d.ptr(b), staged.back().data(),
                                     staged.back().size() * sizeof(int32_t), stream);
    if (rc != MI355X_OK) return rc;
  }
  return MI355X_OK;
}
// Whether any lookup of `fn` takes its bag positions from placeholder `name`.
bool derivesFrom(const MI355XFunction &fn, const std::string &name) {
  for (const auto &d : fn.derivedBagOffsets)
    if (d.lengths == name) return true;
  return false;
}
} // namespace

namespace {
Error fromStatus(int rc, const char *what) {
  if (rc == MI355X_OK) return Error::success();
  ErrorCode c = ErrorCode::RUNTIME_ERROR;
  if (rc == MI355X_ERR_OUT_OF_DEVICE_MEMORY) c = ErrorCode::RUNTIME_OUT_OF_DEVICE_MEMORY;
  else if (rc == MI355X_ERR_NOT_SUPPORTED) c = ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED;
  else if (rc == MI355X_ERR_DEVICE_NOT_FOUND) c = ErrorCode::RUNTIME_DEVICE_NOT_FOUND;
  return MI355X_MAKE_ERR(c, "%s: %s", what, mi355x_last_error());
}
} // namespace

MI355XDeviceManager::~MI355XDeviceManager() { (void)stop(true); }

void MI355XDeviceManager::enqueue(std::function<void()> work) {
  {
    std::lock_guard<std::mutex> lk(mu_);
    queue_.push_back(std::move(work));
  }
  cv_.notify_one();
}

void MI355XDeviceManager::workerLoop() {
  for (;;) {
    std::function<void()> work;
    {
      std::unique_lock<std::mutex> lk(mu_);
      cv_.wait(lk, [this] { return stopping_ || !queue_.empty(); });
      if (queue_.empty()) return; // stopping and drained
      work = std::move(queue_.front());
      queue_.pop_front();
    }
    work();
  }
}

Error MI355XDeviceManager::init() {
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (running_) return Error::success();
    running_ = true;
    stopping_ = false;
  }
  worker_ = std::thread([this] { workerLoop(); });
  // the device is bound to the worker thread, so bind it there
  std::promise<Error> done;
  auto fut = done.get_future();
  enqueue([this, &done] {
    int n = 0;
    if (mi355x_num_devices(&n) != MI355X_OK || config_.deviceID < 0 || config_.deviceID >= n) {
      done.set_value(MI355X_MAKE_ERR(ErrorCode::RUNTIME_DEVICE_NOT_FOUND,
                                     "no MI355X device %d (%d visible)", config_.deviceID, n));
      return;
    }
    int rc = mi355x_init(config_.deviceID);
    if (rc != MI355X_OK) {
      done.set_value(MI355X_MAKE_ERR(ErrorCode::RUNTIME_DEVICE_NOT_FOUND, "%s", mi355x_last_error()));
      return;
    }
    mi355x_info info;
    rc = mi355x_device_info(&info);
    if (rc == MI355X_OK) rc = mi355x_stream_create(&stream_);
    for (int i = 1; i < config_.graphBranches && rc == MI355X_OK; i++) {
      void *s = nullptr;
      rc = mi355x_stream_create(&s);
      if (rc == MI355X_OK) sideStreams_.push_back(s);
    }
    if (rc != MI355X_OK) {
      done.set_value(fromStatus(rc, "device set-up"));
      return;
    }
    info_.name = info.name;
    info_.arch = info.arch;
    info_.totalMemory = info.total_memory;
    info_.computeUnits = info.compute_units;
    maxMemoryBytes_ = config_.deviceMemory ? config_.deviceMemory : info.free_memory;
    done.set_value(Error::success());
  });
  Error e = fut.get();
  if (e) (void)stop(true);
  return e;
}

Error MI355XDeviceManager::stop(bool block) {
  (void)block;
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_) return Error::success();
  }
  std::promise<void> done;
  auto fut = done.get_future();
  enqueue([this, &done] {
    for (auto &kv : functions_) release(kv.second);
    functions_.clear();
    for (auto &kv : modules_)
      if (kv.second.arena) mi355x_arena_destroy(kv.second.arena);
    modules_.clear();
    usedMemoryBytes_ = 0;
    if (stream_) {
      mi355x_stream_sync(stream_);
      mi355x_stream_destroy(stream_);
      stream_ = nullptr;
    }
    for (void *s : sideStreams_) mi355x_stream_destroy(s);
    sideStreams_.clear();
    done.set_value();
  });
  fut.get();
  {
    std::lock_guard<std::mutex> lk(mu_);
    stopping_ = true;
  }
  cv_.notify_all();
  if (worker_.joinable()) worker_.join();
  {
    std::lock_guard<std::mutex> lk(mu_);
    running_ = false;
  }
  return Error::success();
}

void MI355XDeviceManager::addNetwork(const Module *module, FunctionMapTy functions,
                                     ReadyCBTy readyCB) {
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_ || stopping_) {
      readyCB(module, MI355X_MAKE_ERR(ErrorCode::RUNTIME_REQUEST_REFUSED,
                                      "device manager is not running"));
      return;
    }
  }
  enqueue([this, module, functions, readyCB]() mutable {
    addNetworkImpl(module, std::move(functions), std::move(readyCB));
  });
}

void MI355XDeviceManager::evictNetwork(std::string functionName, EvictFunctionCBTy evictCB) {
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_ || stopping_) {
      evictCB(functionName, MI355X_MAKE_ERR(ErrorCode::RUNTIME_REQUEST_REFUSED,
                                            "device manager is not running"));
      return;
    }
  }
  enqueue([this, functionName, evictCB]() mutable {
    evictNetworkImpl(std::move(functionName), std::move(evictCB));
  });
}

RunIdentifierTy MI355XDeviceManager::runFunction(std::string functionName,
                                                 std::unique_ptr<ExecutionContext> ctx,
                                                 ResultCBTy resultCB) {
  const RunIdentifierTy id = nextRun_++;
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_ || stopping_) {
      resultCB(id, MI355X_MAKE_ERR(ErrorCode::RUNTIME_REQUEST_REFUSED,
                                   "device manager is not running"),
               std::move(ctx));
      return id;
    }
  }
  // std::function needs copyable captures: hand the context over by raw pointer
  ExecutionContext *raw = ctx.release();
  enqueue([this, id, functionName, raw, resultCB]() mutable {
    runFunctionImpl(id, std::move(functionName), std::unique_ptr<ExecutionContext>(raw),
                    std::move(resultCB));
  });
  return id;
}

void MI355XDeviceManager::transferStaticPlaceholderToDevice(
    const Module *module, std::string placeholderName, Tensor *tensor,
    std::function<void(Error)> resultCB) {
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_ || stopping_) {
      resultCB(MI355X_MAKE_ERR(ErrorCode::RUNTIME_REQUEST_REFUSED, "device manager is not running"));
      return;
    }
  }
  enqueue([this, module, placeholderName, tensor, resultCB] {
    auto mit = modules_.find(module);
    if (!module || mit == modules_.end() || !mit->second.arena || !tensor) {
      resultCB(MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR,
                               "cannot copy placeholder %s: its module has no function on this device",
                               placeholderName.c_str()));
      return;
    }
    const int id = module->getValueByName(placeholderName);
    if (id < 0 || module->value(id).category != SymbolCategory::Placeholder) {
      resultCB(MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "%s is not a placeholder of the module",
                               placeholderName.c_str()));
      return;
    }
    const Value &v = module->value(id);
    if (tensor->sizeInBytes() > v.type.sizeInBytes()) {
      resultCB(MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "tensor for %s has %zu bytes, slot %zu",
                               placeholderName.c_str(), tensor->sizeInBytes(), v.type.sizeInBytes()));
      return;
    }
    int rc = mi355x_arena_upload(mit->second.arena, MI355X_REGION_MUTABLE, v.offset, tensor->data(),
                                 tensor->sizeInBytes(), stream_);
    // lookups of the module's functions that take their bags from this placeholder
    std::vector<std::vector<int32_t>> staged;
    if (rc == MI355X_OK) {
      void *slot = nullptr;
      mi355x_arena_ptr(mit->second.arena, MI355X_REGION_MUTABLE, v.offset, &slot);
      rc = lengthsUploaded(module, placeholderName, (uint8_t *)slot, v.type.sizeInBytes(),
                           tensor->data(), tensor->sizeInBytes(), staged);
    }
    if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
    resultCB(rc == MI355X_OK ? Error::success() : fromStatus(rc, "placeholder copy"));
  });
}

Expected<float> MI355XDeviceManager::timeFunction(const std::string &functionName, int iterations) {
  {
    std::lock_guard<std::mutex> lk(mu_);
    if (!running_ || stopping_)
      return MI355X_MAKE_ERR(ErrorCode::RUNTIME_REQUEST_REFUSED, "device manager is not running");
  }
  if (iterations < 1)
    return MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "iterations must be positive");
  std::promise<std::pair<Error, float>> done;
  auto fut = done.get_future();
  enqueue([this, &done, functionName, iterations] {
    auto it = functions_.find(functionName);
    if (it == functions_.end()) {
      done.set_value({MI355X_MAKE_ERR(ErrorCode::RUNTIME_NET_NOT_FOUND, "Function %s not found",
                                      functionName.c_str()),
                      0.0f});
      return;
    }
    FunctionResident &fr = it->second;
    ExecutionContext ctx;
    ctx.setDeviceBindings(std::unique_ptr<DeviceBindings>(new DeviceBindings(fr.bindings)));
    void *e0 = nullptr, *e1 = nullptr;
    Error err;
    float ms = 0.0f;
    // the comparison of recordings, if still going on, finishes untimed
    while (!fr.branchesTuned && !err) err = executeTuned(fr, &ctx);
    int rc = mi355x_event_create(&e0);
    if (rc == MI355X_OK) rc = mi355x_event_create(&e1);
    if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
    if (rc == MI355X_OK) rc = mi355x_event_record(e0, stream_);
    if (rc != MI355X_OK && !err) err = fromStatus(rc, "timing set-up");
    for (int i = 0; i < iterations && !err; i++) err = fr.fn->execute(&ctx);
    if (!err) {
      rc = mi355x_event_record(e1, stream_);
      if (rc == MI355X_OK) rc = mi355x_event_sync(e1);
      if (rc == MI355X_OK) rc = mi355x_event_elapsed_ms(e0, e1, &ms);
      if (rc != MI355X_OK) err = fromStatus(rc, "timing");
    }
    mi355x_stream_sync(stream_);
    if (e0) mi355x_event_destroy(e0);
    if (e1) mi355x_event_destroy(e1);
    done.set_value({std::move(err), ms / (float)iterations});
  });
  auto r = fut.get();
  if (r.first) return r.first;
  return r.second;
}

void MI355XDeviceManager::release(FunctionResident &fr) {
  if (fr.fn) fr.fn->dropGraph();
  if (fr.arena) mi355x_arena_destroy(fr.arena);
  fr.arena = nullptr;
  usedMemoryBytes_ -= fr.bytes;
  auto it = modules_.find(fr.module);
  if (it != modules_.end() && --it->second.users == 0) {
    if (it->second.arena) mi355x_arena_destroy(it->second.arena);
    usedMemoryBytes_ -= it->second.bytes;
    modules_.erase(it);
  }
}

// `bytes` of placeholder `name` of `module` have just been copied into its slot
// (slotBytes long). If lookups of any resident function of the module take
// their bag positions from it, the rest of the slot is cleared (a partial
// tensor: the missing bags are empty for the kernels that read the lengths and
// for the positions alike) and every such function's positions are refreshed:
// the slot belongs to the module, so a function that is not the one being run
// must not keep positions of the lengths it held before.
int MI355XDeviceManager::lengthsUploaded(const Module *module, const std::string &name,
                                         uint8_t *slot, size_t slotBytes, const void *data,
                                         size_t bytes,
                                         std::vector<std::vector<int32_t>> &staged) {
  bool derived = false;
  for (auto &f : functions_)
    if (f.second.module == module && derivesFrom(*f.second.fn, name)) derived = true;
  if (!derived) return MI355X_OK;
  int rc = MI355X_OK;
  if (bytes < slotBytes) rc = mi355x_fill_u8(slot + bytes, 0, slotBytes - bytes, stream_);
  for (auto &f : functions_)
    if (rc == MI355X_OK && f.second.module == module)
      rc = uploadBagOffsets(*f.second.fn, f.second.bindings, name, data, bytes, stream_, staged);
  return rc;
}

Error MI355XDeviceManager::makeResident(const Module *module, const std::string &name,
                                        MI355XFunction *fn) {
  const RuntimeBundle &rb = fn->getRuntimeBundle();
  // A function that writes a placeholder on the device and one that derives bag
  // positions from the host's copy of the same placeholder cannot share a module.
  for (const auto &f : functions_) {
    if (f.second.module != module) continue;
    for (const auto &w : fn->writtenPlaceholders)
      if (derivesFrom(*f.second.fn, w))
        return MI355X_MAKE_ERR(ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED,
                               "function %s writes placeholder %s, from which resident function "
                               "%s takes bag positions made on the host: compile that one with "
                               "deriveBagOffsets off",
                               name.c_str(), w.c_str(), f.first.c_str());
    for (const auto &w : f.second.fn->writtenPlaceholders)
      if (derivesFrom(*fn, w))
        return MI355X_MAKE_ERR(ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED,
                               "function %s takes bag positions made on the host from placeholder "
                               "%s, which resident function %s writes: compile it with "
                               "deriveBagOffsets off",
                               name.c_str(), w.c_str(), f.first.c_str());
  }
  ModuleResident &mr = modules_[module];
  if (!mr.arena && mr.users == 0) {
    int rc = mi355x_arena_create(module->constantsSize(), module->mutableSize(), 0, &mr.arena);
    if (rc != MI355X_OK) {
      modules_.erase(module);
      return fromStatus(rc, "module arena");
    }
    mr.bytes = mi355x_arena_bytes(mr.arena);
    usedMemoryBytes_ += mr.bytes;
    // placeholders start as zeros: the first (untimed) pass over a new network
    // runs before any request has filled them
    if (module->mutableSize()) {
      void *mp = nullptr;
      mi355x_arena_ptr(mr.arena, MI355X_REGION_MUTABLE, 0, &mp);
      mi355x_fill_u8(mp, 0, module->mutableSize(), stream_);
    }
    if (module->constantsSize()) {
      rc = mi355x_arena_upload(mr.arena, MI355X_REGION_CONSTANTS, 0,
                               module->constantsImage().data(), module->constantsSize(), stream_);
      if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
      if (rc != MI355X_OK) {
        mi355x_arena_destroy(mr.arena);
        usedMemoryBytes_ -= mr.bytes;
        modules_.erase(module);
        return fromStatus(rc, "constants upload");
      }
    }
  }
  mr.users++;
  FunctionResident fr;
  fr.fn = fn;
  fr.module = module;
  auto failWith = [&](Error e) {
    release(fr);
    return e;
  };
  int rc = mi355x_arena_create(rb.generatedConstantsMemSize, 0, rb.activationsMemSize, &fr.arena);
  if (rc != MI355X_OK) return failWith(fromStatus(rc, "function arena"));
  fr.bytes = mi355x_arena_bytes(fr.arena);
  usedMemoryBytes_ += fr.bytes;
  if (rb.activationsMemSize) {
    void *ap = nullptr;
    mi355x_arena_ptr(fr.arena, MI355X_REGION_ACTIVATIONS, 0, &ap);
    mi355x_fill_u8(ap, 0, rb.activationsMemSize, stream_);
  }
  void *p = nullptr;
  mi355x_arena_ptr(mr.arena, MI355X_REGION_CONSTANTS, 0, &p);
  fr.bindings.constants = (uint8_t *)p;
  mi355x_arena_ptr(mr.arena, MI355X_REGION_MUTABLE, 0, &p);
  fr.bindings.mutableMem = (uint8_t *)p;
  mi355x_arena_ptr(fr.arena, MI355X_REGION_CONSTANTS, 0, &p);
  fr.bindings.generated = (uint8_t *)p;
  mi355x_arena_ptr(fr.arena, MI355X_REGION_ACTIVATIONS, 0, &p);
  fr.bindings.activations = (uint8_t *)p;
  fr.bindings.stream = stream_;
  fr.bindings.opts.slws_math = config_.slwsMath;
  if (!fn->generated.empty()) {
    rc = mi355x_arena_upload(fr.arena, MI355X_REGION_CONSTANTS, 0, fn->generated.data(),
                             fn->generated.size(), stream_);
    if (rc != MI355X_OK) return failWith(fromStatus(rc, "generated constants upload"));
  }
  // bag positions of lookups that take them from the host: from what the
  // lengths placeholders hold right now (zeros on a new module)
  for (const auto &d : fn->derivedBagOffsets) {
    auto st = rb.symbolTable.find(d.lengths);
    if (st == rb.symbolTable.end()) continue;
    std::vector<int32_t> cur(d.segments, 0);
    rc = mi355x_memcpy_d2h(cur.data(), fr.bindings.mutableMem + st->second.offset,
                           d.segments * sizeof(int32_t), stream_);
    if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
    std::vector<std::vector<int32_t>> staged;
    if (rc == MI355X_OK)
      rc = uploadBagOffsets(*fn, fr.bindings, d.lengths, cur.data(), cur.size() * sizeof(int32_t),
                            stream_, staged);
    if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
    if (rc != MI355X_OK) return failWith(fromStatus(rc, "bag offsets"));
  }
  for (const auto &l : fn->setup) {
    rc = l.run(fr.bindings);
    if (rc != MI355X_OK) return failWith(fromStatus(rc, l.kernel.c_str()));
  }
  rc = mi355x_stream_sync(stream_);
  if (rc != MI355X_OK) return failWith(fromStatus(rc, "set-up launches"));
  if (config_.useLaunchGraphs) {
    // one eager pass first: entry points that allocate on first use must have
    // run before they are recorded
    for (const auto &l : fn->launches) {
      rc = l.launch(fr.bindings);
      if (rc != MI355X_OK) return failWith(fromStatus(rc, l.kernel.c_str()));
    }
    rc = mi355x_stream_sync(stream_);
    if (rc != MI355X_OK) return failWith(fromStatus(rc, "first pass"));
    if (config_.autotuneTiles) {
      Error te = tuneTiles(fn, fr.bindings);
      if (te) return failWith(std::move(te));
    }
    Error e = fn->captureGraph(fr.bindings, sideStreams_);
    if (e) return failWith(std::move(e));
    const int all = (int)sideStreams_.size() + 1;
    if (config_.autotuneBranches && all > 1) {
      fr.branchCandidates = {all, 1};
      if (all > 2) fr.branchCandidates.push_back(2);
      fr.branchesTuned = false;
    }
  }
  functions_.emplace(name, fr);
  return Error::success();
}

Error MI355XDeviceManager::captureWithBranches(FunctionResident &fr, int branches) {
  std::vector<void *> side(sideStreams_.begin(),
                           sideStreams_.begin() + std::min<size_t>(sideStreams_.size(),
                                                                   (size_t)std::max(0, branches - 1)));
  return fr.fn->captureGraph(fr.bindings, side);
}

// Runs one request. While the recordings of a function are still being
// compared it also re-records and times as the phase says; every request
// computes the same results whichever recording replays it.
Error MI355XDeviceManager::executeTuned(FunctionResident &fr, ExecutionContext *ctx) {
  if (fr.branchesTuned) return fr.fn->execute(ctx);
  constexpr int kPerCandidate = 3;       // one warm-up and two timed requests
  const size_t cand = (size_t)(fr.branchPhase / kPerCandidate);
  const bool timed = fr.branchPhase % kPerCandidate != 0;
  Error err;
  if (!timed) {
    // candidate 0 is the recording made at load time
    if (cand > 0) err = captureWithBranches(fr, fr.branchCandidates[cand]);
    if (!err) err = fr.fn->execute(ctx);
  } else {
    void *e0 = nullptr, *e1 = nullptr;
    float ms = 0.0f;
    int rc = mi355x_event_create(&e0);
    if (rc == MI355X_OK) rc = mi355x_event_create(&e1);
    if (rc == MI355X_OK) rc = mi355x_stream_sync(stream_);
    if (rc == MI355X_OK) rc = mi355x_event_record(e0, stream_);
    if (rc == MI355X_OK) {
      err = fr.fn->execute(ctx);
      if (!err) {
        rc = mi355x_event_record(e1, stream_);
        if (rc == MI355X_OK) rc = mi355x_event_sync(e1);
        if (rc == MI355X_OK) rc = mi355x_event_elapsed_ms(e0, e1, &ms);
      }
    }
    if (e0) mi355x_event_destroy(e0);
    if (e1) mi355x_event_destroy(e1);
    if (!err && rc != MI355X_OK) err = fromStatus(rc, "branch timing");
    if (!err) {
      if (fr.branchMs.size() <= cand) fr.branchMs.push_back(ms);
      else fr.branchMs[cand] = std::min(fr.branchMs[cand], ms);
    }
  }
  if (err) {
    // fall back to the recording with all branches and stop comparing
    fr.branchesTuned = true;
    Error again = captureWithBranches(fr, fr.branchCandidates[0]);
    (void)again;
    return err;
  }
  if (++fr.branchPhase == kPerCandidate * (int)fr.branchCandidates.size()) {
    size_t best = 0;
    for (size_t i = 1; i < fr.branchMs.size(); i++)
      if (fr.branchMs[i] < fr.branchMs[best]) best = i;
    fr.branchesTuned = true;
    if (best + 1 != fr.branchCandidates.size())
      return captureWithBranches(fr, fr.branchCandidates[best]);
  }
  return Error::success();
}

// For every matrix-core launch: run each tile a few times on the resident data
// and keep the fastest (results do not depend on the tile).
Error MI355XDeviceManager::tuneTiles(MI355XFunction *fn, const DeviceBindings &b) {
  void *e0 = nullptr, *e1 = nullptr;
  int rc = mi355x_event_create(&e0);
  if (rc == MI355X_OK) rc = mi355x_event_create(&e1);
  Error err;
  // A launch of a few microseconds cannot be told from its neighbour by four
  // runs between two events: every candidate gets two series of kRuns launches
  // and its faster series counts. Three passes over the whole function first
  // bring the clocks up, so the first candidates are not timed on an idle part.
  constexpr int kRuns = 16, kSeries = 2;
  for (int pass = 0; pass < 3 && rc == MI355X_OK; pass++)
    for (auto &l : fn->launches)
      if (rc == MI355X_OK) rc = l.launch(b);
  // seconds of kRuns launches of launch l with tile t (the faster of kSeries
  // series); negative when the tile cannot serve the launch
  auto timeTile = [&](KernelLaunch &l, int t) -> float {
    l.tile = t;
    if (l.launch(b) != MI355X_OK) return -1.0f;   // warm-up, also rejects tiles the shape cannot use
    float ms = 0.0f;
    for (int s = 0; s < kSeries && rc == MI355X_OK; s++) {
      rc = mi355x_event_record(e0, stream_);
      for (int i = 0; i < kRuns && rc == MI355X_OK; i++) rc = l.launch(b);
      if (rc == MI355X_OK) rc = mi355x_event_record(e1, stream_);
      if (rc == MI355X_OK) rc = mi355x_event_sync(e1);
      float one = 0.0f;
      if (rc == MI355X_OK) rc = mi355x_event_elapsed_ms(e0, e1, &one);
      if (s == 0 || one < ms) ms = one;
    }
    return ms;
  };
  for (auto &l : fn->launches) {
    if (!l.tunable || rc != MI355X_OK) continue;
    float best = 0.0f;
    int bestTile = -1;
    for (int t = -1; t < kNumTiles && rc == MI355X_OK; t++) {
      const float ms = timeTile(l, t);
      if (ms < 0.0f) continue;
      if (rc == MI355X_OK && (t == -1 || ms < best)) {
        best = ms;
        bestTile = t;
      }
    }
    // A dozen candidates a few per cent apart: the fastest of one pass is often
    // a lucky measurement (several tile numbers run the very kernel the shape
    // rule picks). The winner has to beat the library's own choice again, by
    // two per cent, in a second pass, or that choice stays.
    if (bestTile != -1 && rc == MI355X_OK) {
      const float again = timeTile(l, bestTile), base = timeTile(l, -1);
      if (!(again >= 0.0f && base >= 0.0f && again < 0.98f * base)) bestTile = -1;
    }
    l.tile = bestTile;
  }
  if (rc != MI355X_OK) err = fromStatus(rc, "tile tuning");
  if (e0) mi355x_event_destroy(e0);
  if (e1) mi355x_event_destroy(e1);
  mi355x_stream_sync(stream_);
  return err;
}

void MI355XDeviceManager::addNetworkImpl(const Module *module, FunctionMapTy functions,
                                         ReadyCBTy readyCB) {
  uint64_t need = 0;
  for (const auto &f : functions) {
    if (functions_.count(f.first)) {
      readyCB(module, MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR,
                                      "Failed to add network: already have a function called %s",
                                      f.first.c_str()));
      return;
    }
    if (!f.second || f.second->getCompileBackendName() != "MI355X") {
      readyCB(module, MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR,
                                      "Failed to add network: function %s is not an MI355XFunction",
                                      f.first.c_str()));
      return;
    }
    const RuntimeBundle &rb = f.second->getRuntimeBundle();
    need += rb.generatedConstantsMemSize + rb.activationsMemSize;
  }
  if (!modules_.count(module)) need += module->constantsSize() + module->mutableSize();
  if (usedMemoryBytes_ + need > maxMemoryBytes_) {
    readyCB(module, MI355X_MAKE_ERR(ErrorCode::RUNTIME_OUT_OF_DEVICE_MEMORY,
                                    "Failed to add network: not enough memory (%llu needed, "
                                    "%llu available)",
                                    (unsigned long long)need,
                                    (unsigned long long)(maxMemoryBytes_ - usedMemoryBytes_)));
    return;
  }
  std::vector<std::string> added;
  for (const auto &f : functions) {
    Error e = makeResident(module, f.first, f.second);
    if (e) {
      for (const auto &n : added) {
        release(functions_[n]);
        functions_.erase(n);
      }
      readyCB(module, std::move(e));
      return;
    }
    added.push_back(f.first);
  }
  readyCB(module, Error::success());
}

void MI355XDeviceManager::evictNetworkImpl(std::string functionName, EvictFunctionCBTy evictCB) {
  auto it = functions_.find(functionName);
  if (it == functions_.end()) {
    evictCB(functionName, MI355X_MAKE_ERR(ErrorCode::RUNTIME_NET_NOT_FOUND,
                                          "Could not find function with name %s to evict",
                                          functionName.c_str()));
    return;
  }
  mi355x_stream_sync(stream_);
  release(it->second);
  functions_.erase(it);
  evictCB(functionName, Error::success());
}

void MI355XDeviceManager::runFunctionImpl(RunIdentifierTy id, std::string functionName,
                                          std::unique_ptr<ExecutionContext> ctx,
                                          ResultCBTy resultCB) {
  auto it = functions_.find(functionName);
  if (it == functions_.end()) {
    resultCB(id, MI355X_MAKE_ERR(ErrorCode::RUNTIME_NET_NOT_FOUND, "Function %s not found",
                                 functionName.c_str()),
             std::move(ctx));
    return;
  }
  if (!ctx) {
    resultCB(id, MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "no execution context"), nullptr);
    return;
  }
  FunctionResident &fr = it->second;
  const RuntimeBundle &rb = fr.fn->getRuntimeBundle();
  PlaceholderBindings *pb = ctx->getPlaceholderBindings();
  Error err;
  std::vector<std::vector<int32_t>> staged; // bag positions on their way to the device
  // inputs: host tensor -> placeholder slot (a tensor smaller than the slot
  // fills its front, like the reference's partial tensors)
  for (const auto &kv : pb->pairs()) {
    auto st = rb.symbolTable.find(kv.first);
    if (st == rb.symbolTable.end() || st->second.symbolCategory != SymbolCategory::Placeholder)
      continue;
    if (!st->second.input || !kv.second) continue;
    if (kv.second->sizeInBytes() > st->second.size) {
      err = MI355X_MAKE_ERR(ErrorCode::RUNTIME_ERROR, "tensor bound to %s has %zu bytes, slot %zu",
                            kv.first.c_str(), kv.second->sizeInBytes(), st->second.size);
      break;
    }
    int rc = mi355x_memcpy_h2d(fr.bindings.mutableMem + st->second.offset, kv.second->data(),
                               kv.second->sizeInBytes(), stream_);
    if (rc == MI355X_OK)
      rc = lengthsUploaded(fr.module, kv.first, fr.bindings.mutableMem + st->second.offset,
                           st->second.size, kv.second->data(), kv.second->sizeInBytes(), staged);
    if (rc != MI355X_OK) {
      err = fromStatus(rc, "input copy");
      break;
    }
  }
  if (!err) {
    ctx->setDeviceBindings(std::unique_ptr<DeviceBindings>(new DeviceBindings(fr.bindings)));
    err = executeTuned(fr, ctx.get());
  }
  if (!err) {
    for (const auto &kv : pb->pairs()) {
      auto st = rb.symbolTable.find(kv.first);
      if (st == rb.symbolTable.end() || st->second.symbolCategory != SymbolCategory::Placeholder)
        continue;
      if (!st->second.output || !kv.second) continue;
      const size_t n = std::min(kv.second->sizeInBytes(), st->second.size);
      int rc = mi355x_memcpy_d2h(kv.second->data(), fr.bindings.mutableMem + st->second.offset, n,
                                 stream_);
      if (rc != MI355X_OK) {
        err = fromStatus(rc, "output copy");
        break;
      }
    }
  }
  const int rc = mi355x_stream_sync(stream_);
  if (!err && rc != MI355X_OK) err = fromStatus(rc, "run");
  resultCB(id, std::move(err), std::move(ctx));
}

} // namespace glow_mi355x

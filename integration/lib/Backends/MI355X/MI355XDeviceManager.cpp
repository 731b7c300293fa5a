/**
 * MI355XDeviceManager: one MI355X as a Glow runtime device.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/Backends/DeviceManager.h,
 * QueueBackedDeviceManager.h and the behaviour of
 * lib/Backends/CPU/CPUDeviceManager.cpp:65-177 (name checks, memory check,
 * error codes) and lib/Backends/OpenCL/OpenCLDeviceManager.cpp:775-845 (inputs
 * to the device, execute, outputs back, one callback).
 */
#include "MI355XDeviceManager.h"
#include "MI355XFunction.h"

#include "glow/Graph/PlaceholderBindings.h"
#include "glow/Support/Error.h"

#include "glow_mi355x.h"

#include "llvm/Support/FormatVariadic.h"

#include <future>

using namespace glow;
using namespace glow::runtime;

namespace hm = glow_mi355x;

DeviceManager *glow::runtime::createMI355XDeviceManager(const DeviceConfig &config) {
  return new MI355XDeviceManager(config);
}

MI355XDeviceManager::MI355XDeviceManager(const DeviceConfig &config)
    : QueueBackedDeviceManager(config) {}

MI355XDeviceManager::~MI355XDeviceManager() {
  ERR_TO_VOID(stop(true));
  for (void *p : pinned_) {
    mi355x_host_free(p);
  }
}

Error MI355XDeviceManager::init() {
  hm::DeviceConfig hc;
  hc.deviceID = static_cast<int>(config_.deviceID);
  hc.deviceMemory = config_.getDeviceMemory(0); // 0: what the device has free
  // DeviceConfig::parameters: "graphs" = 0 replays kernel by kernel,
  // "branches" = n records at most n parallel branches per function
  if (getParamByName("graphs") == "0") {
    hc.useLaunchGraphs = false;
  }
  if (!getParamByName("branches").empty()) {
    hc.graphBranches = std::max(1, std::stoi(getParamByName("branches").str()));
  }
  impl_ = glow::make_unique<hm::MI355XDeviceManager>(hc);
  RETURN_IF_ERR(toGlowError(impl_->init()));
  maxMemoryBytes_ = impl_->getMaximumMemory();
  exportMemoryCounters();
  return Error::success();
}

Error MI355XDeviceManager::stop(bool block) {
  Error e = QueueBackedDeviceManager::stop(block);
  if (impl_) {
    Error e2 = toGlowError(impl_->stop(true));
    if (!e) {
      e = std::move(e2);
    } else {
      ERR_TO_VOID(std::move(e2));
    }
  }
  zeroMemoryCounters();
  return e;
}

uint64_t MI355XDeviceManager::getMaximumMemory() const {
  return impl_ ? impl_->getMaximumMemory() : 0;
}
uint64_t MI355XDeviceManager::getAvailableMemory() const {
  return impl_ ? impl_->getAvailableMemory() : 0;
}
bool MI355XDeviceManager::isMemoryAvailable(uint64_t estimate) const {
  return impl_ && impl_->isMemoryAvailable(estimate);
}

DeviceInfo MI355XDeviceManager::getDeviceInfo() const {
  // Published MI355X figures, in the units the partitioner expects.
  DeviceInfo info = DeviceInfo();
  info.availableMemory = getAvailableMemory();
  info.backendName = "MI355X";
  info.sramCapacity = 256ull * 1024 * 1024;          // Infinity Cache
  info.peakCompute = 5.0e15;                          // dense int8 op/s
  info.peakDramBw = 8.0e12;                           // HBM3E bytes/s
  info.peakSramBw = 14.0e12;
  info.peakPCIeBw = 64.0e9;
  return info;
}

void *MI355XDeviceManager::allocateDeviceIOBuffer(dim_t size) {
  std::lock_guard<std::mutex> lock(bufferLock_);
  void *p = nullptr;
  if (mi355x_host_alloc(&p, size) != MI355X_OK) {
    return nullptr;
  }
  pinned_.insert(p);
  return p;
}

void MI355XDeviceManager::freeAllocatedDeviceIOBuffer(void *buffer) {
  std::lock_guard<std::mutex> lock(bufferLock_);
  auto it = pinned_.find(buffer);
  if (it != pinned_.end()) {
    mi355x_host_free(buffer);
    pinned_.erase(it);
  }
}

void MI355XDeviceManager::addNetworkImpl(const Module *module,
                                         FunctionMapTy functions,
                                         ReadyCBTy readyCB) {
  DCHECK(readyCB != nullptr);
  for (const auto &func : functions) {
    if (functions_.count(func.first) != 0) {
      readyCB(module,
              MAKE_ERR(llvm::formatv("Failed to add network: already have a "
                                     "function called {0}",
                                     func.first)
                           .str()));
      return;
    }
    if (func.second->getCompileBackendName() != "MI355X") {
      readyCB(module,
              MAKE_ERR(llvm::formatv("Failed to add network: function {0} is "
                                     "not an MI355XFunction",
                                     func.first)
                           .str()));
      return;
    }
  }
  // One host-layer addNetwork per function: every MI355XFunction was compiled
  // against its own restated module (constants copied at compile time), and
  // the host manager keys residency by that module.
  std::vector<std::string> added;
  for (const auto &func : functions) {
    auto *mf = static_cast<MI355XFunction *>(func.second);
    std::promise<hm::Error> done;
    auto fut = done.get_future();
    hm::FunctionMapTy one;
    one[func.first] = mf->hostFunction();
    impl_->addNetwork(mf->hostModule(), one,
                      [&done](const hm::Module *, hm::Error e) {
                        done.set_value(std::move(e));
                      });
    hm::Error e = fut.get();
    if (e) {
      for (const auto &name : added) {
        std::promise<void> ev;
        auto evf = ev.get_future();
        impl_->evictNetwork(name, [&ev](std::string, hm::Error) { ev.set_value(); });
        evf.get();
        functions_.erase(name);
      }
      readyCB(module, toGlowError(e));
      return;
    }
    added.push_back(func.first);
    functions_[func.first] = Resident{func.second, module};
  }
  usedMemoryBytes_ = impl_->getMaximumMemory() - impl_->getAvailableMemory();
  exportMemoryCounters();
  readyCB(module, Error::success());
}

void MI355XDeviceManager::evictNetworkImpl(std::string functionName,
                                           EvictFunctionCBTy evictCB) {
  DCHECK(evictCB != nullptr);
  if (functions_.erase(functionName) == 0) {
    evictCB(functionName,
            MAKE_ERR(ErrorValue::ErrorCode::RUNTIME_NET_NOT_FOUND,
                     strFormat("Could not find function with name %s to evict",
                               functionName.c_str())));
    return;
  }
  std::promise<hm::Error> done;
  auto fut = done.get_future();
  impl_->evictNetwork(functionName, [&done](std::string, hm::Error e) {
    done.set_value(std::move(e));
  });
  hm::Error e = fut.get();
  usedMemoryBytes_ = impl_->getMaximumMemory() - impl_->getAvailableMemory();
  exportMemoryCounters();
  evictCB(functionName, toGlowError(e));
}

void MI355XDeviceManager::runFunctionImpl(RunIdentifierTy id,
                                          std::string functionName,
                                          std::unique_ptr<ExecutionContext> context,
                                          ResultCBTy resultCB) {
  DCHECK(resultCB != nullptr);
  TRACE_EVENT_SCOPE_NAMED(context->getTraceContext(), TraceLevel::RUNTIME,
                          "DeviceManager::run", dmRun);
  if (functions_.find(functionName) == functions_.end()) {
    dmRun.addArg("reason", "function not found");
    TRACE_EVENT_SCOPE_END_NAMED(dmRun);
    resultCB(id,
             MAKE_ERR(ErrorValue::ErrorCode::RUNTIME_NET_NOT_FOUND,
                      llvm::formatv("Function {0} not found", functionName).str()),
             std::move(context));
    return;
  }
  // Host tensors by placeholder name, borrowed for the duration of the run.
  // A partial tensor (Tensor::getUnpaddedSizeInBytes) fills the front of its
  // slot, as the reference's partial-tensor contract says.
  context->getPlaceholderBindings()->ensureOnHost();
  auto hostCtx = std::unique_ptr<hm::ExecutionContext>(new hm::ExecutionContext());
  std::vector<hm::Tensor> borrowed;
  borrowed.reserve(context->getPlaceholderBindings()->pairs().size());
  for (auto &kv : context->getPlaceholderBindings()->pairs()) {
    Tensor &t = kv.second;
    const size_t bytes = t.getUnpaddedSizeInBytes();
    borrowed.push_back(hm::Tensor::unowned(
        hm::Type(hm::ElemKind::Int8QTy, {(int64_t)bytes}), t.getUnsafePtr(), bytes));
    hostCtx->getPlaceholderBindings()->insert(kv.first->getName().str(),
                                              &borrowed.back());
  }
  std::promise<hm::Error> done;
  auto fut = done.get_future();
  impl_->runFunction(functionName, std::move(hostCtx),
                     [&done](hm::RunIdentifierTy, hm::Error e,
                             std::unique_ptr<hm::ExecutionContext>) {
                       done.set_value(std::move(e));
                     });
  hm::Error e = fut.get();
  TRACE_EVENT_SCOPE_END_NAMED(dmRun);
  // exactly one callback, with the context handed back
  resultCB(id, toGlowError(e), std::move(context));
}

void MI355XDeviceManager::transferStaticPlaceholderToDevice(
    Placeholder *PH, Tensor *T, std::function<void(Error)> resultCB) {
  workThread_.submit([this, PH, T, resultCB = std::move(resultCB)]() mutable {
    if (!PH || !T) {
      resultCB(MAKE_ERR(ErrorValue::ErrorCode::RUNTIME_ERROR,
                        "Invalid Placeholder or Tensor."));
      return;
    }
    // every resident function that knows the placeholder gets the value (each
    // function carries its own restated module)
    bool any = false;
    hm::Tensor borrowed = hm::Tensor::unowned(
        hm::Type(hm::ElemKind::Int8QTy, {(int64_t)T->getUnpaddedSizeInBytes()}),
        T->getUnsafePtr(), T->getUnpaddedSizeInBytes());
    for (auto &kv : functions_) {
      auto *mf = static_cast<MI355XFunction *>(kv.second.function);
      if (mf->hostModule()->getValueByName(PH->getName().str()) < 0) {
        continue;
      }
      std::promise<hm::Error> done;
      auto fut = done.get_future();
      impl_->transferStaticPlaceholderToDevice(
          mf->hostModule(), PH->getName().str(), &borrowed,
          [&done](hm::Error e) { done.set_value(std::move(e)); });
      hm::Error e = fut.get();
      if (e) {
        resultCB(toGlowError(e));
        return;
      }
      any = true;
    }
    if (!any) {
      resultCB(MAKE_ERR(ErrorValue::ErrorCode::RUNTIME_ERROR,
                        strFormat("No resident function uses placeholder %s",
                                  PH->getName().str().c_str())));
      return;
    }
    resultCB(Error::success());
  });
}

/**
 * MI355XDeviceManager: one MI355X as a Glow runtime device.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/Backends/QueueBackedDeviceManager.h.
 */
#ifndef GLOW_BACKENDS_MI355X_MI355XDEVICEMANAGER_H
#define GLOW_BACKENDS_MI355X_MI355XDEVICEMANAGER_H

#include "glow/Backends/QueueBackedDeviceManager.h"
#include "glow/Runtime/RuntimeTypes.h"

// the MI355X host layer (glow_amd/host in the kernel library's repository)
#include "DeviceManager.h"

#include <map>
#include <memory>
#include <string>

namespace glow {
namespace runtime {

class MI355XDeviceManager final : public QueueBackedDeviceManager {
public:
  explicit MI355XDeviceManager(const DeviceConfig &config);
  ~MI355XDeviceManager() override;

  /// Binds the device on the work thread, creates its streams and sets the
  /// memory limit (the DeviceConfig's, or the free HBM).
  Error init() override;
  Error stop(bool block = true) override;

  uint64_t getMaximumMemory() const override;
  uint64_t getAvailableMemory() const override;
  bool isMemoryAvailable(uint64_t estimate) const override;
  DeviceInfo getDeviceInfo() const override;

  /// Pinned host memory, so request tensors reach the device by DMA.
  void *allocateDeviceIOBuffer(dim_t size) override;
  void freeAllocatedDeviceIOBuffer(void *buffer) override;

  /// Copies \p T into the device slot of \p PH once; requests that do not bind
  /// \p PH afterwards read that value.
  void transferStaticPlaceholderToDevice(
      Placeholder *PH, Tensor *T, std::function<void(Error)> resultCB) override;

protected:
  void addNetworkImpl(const Module *module, FunctionMapTy functions,
                      ReadyCBTy readyCB) override;
  void evictNetworkImpl(std::string functionName,
                        EvictFunctionCBTy evictCB) override;
  void runFunctionImpl(RunIdentifierTy id, std::string functionName,
                       std::unique_ptr<ExecutionContext> context,
                       ResultCBTy resultCB) override;

private:
  /// The host layer's manager. It has a work thread of its own; calls from
  /// Glow's work thread block on its callbacks, so Glow's one-at-a-time
  /// contract per device holds unchanged.
  std::unique_ptr<glow_mi355x::MI355XDeviceManager> impl_;
  /// Resident functions: name -> (compiled function, the Glow module it came
  /// from, for static placeholders).
  struct Resident {
    CompiledFunction *function = nullptr;
    const Module *module = nullptr;
  };
  std::map<std::string, Resident> functions_;
  std::set<void *> pinned_;
};

DeviceManager *createMI355XDeviceManager(const DeviceConfig &config);

} // namespace runtime
} // namespace glow

#endif // GLOW_BACKENDS_MI355X_MI355XDEVICEMANAGER_H

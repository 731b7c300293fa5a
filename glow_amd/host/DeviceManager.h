// MI355XDeviceManager: owns one GPU's resident networks and runs them.
// Mirrors glow::runtime::DeviceManager / QueueBackedDeviceManager (reference
// include/glow/Backends/DeviceManager.h:47-241,
// include/glow/Backends/QueueBackedDeviceManager.h:30-127) and the behaviour of
// CPUDeviceManager (lib/Backends/CPU/CPUDeviceManager.cpp:65-177): all work
// runs on one worker thread, results come back through callbacks, errors are
// values.
#ifndef GLOW_MI355X_HOST_DEVICEMANAGER_H
#define GLOW_MI355X_HOST_DEVICEMANAGER_H

#include "Backend.h"

#include <atomic>
#include <condition_variable>
#include <deque>
#include <functional>
#include <map>
#include <mutex>
#include <thread>

struct mi355x_arena;

namespace glow_mi355x {

using RunIdentifierTy = uint64_t;
using FunctionMapTy = std::map<std::string, MI355XFunction *>;
using ReadyCBTy = std::function<void(const Module *, Error)>;
using EvictFunctionCBTy = std::function<void(std::string, Error)>;
using ResultCBTy = std::function<void(RunIdentifierTy, Error, std::unique_ptr<ExecutionContext>)>;

struct DeviceConfig {
  int deviceID = 0;
  uint64_t deviceMemory = 0;  // 0 = what the device reports as free at init
  bool useLaunchGraphs = true; // record each function once, replay per run
  int graphBranches = 4;       // independent launches recorded side by side (1 = a chain)
  bool autotuneTiles = true;   // time the tile candidates of each matrix-core launch at load
  // The first requests of a function replay it recorded with all branches, as
  // one chain and with two branches (a warm-up and two timed requests each); the
  // fastest recording serves the requests after them. Waiting for another
  // stream costs microseconds, so short side branches can lose more than they
  // overlap, and how long a launch runs depends on the request's data.
  bool autotuneBranches = true;
  // Arithmetic of this device manager's SparseLengths launches, passed with
  // every such call (mi355x_launch_opts::slws_math): MI355X_SLWS_MATH_*, or -1
  // for the library's default.
  int slwsMath = -1;
};

struct DeviceInfo {
  std::string name, arch;
  uint64_t totalMemory = 0;
  int computeUnits = 0;
};

class MI355XDeviceManager {
public:
  explicit MI355XDeviceManager(const DeviceConfig &config) : config_(config) {}
  ~MI355XDeviceManager();

  // Starts the worker thread and binds the device; RUNTIME_DEVICE_NOT_FOUND
  // when there is no such gfx950 device.
  Error init();
  // Drains the queue, frees every network, stops the worker.
  Error stop(bool block = true);

  // Asynchronous: the callback runs on the worker thread.
  void addNetwork(const Module *module, FunctionMapTy functions, ReadyCBTy readyCB);
  void evictNetwork(std::string functionName, EvictFunctionCBTy evictCB);
  RunIdentifierTy runFunction(std::string functionName, std::unique_ptr<ExecutionContext> ctx,
                              ResultCBTy resultCB);

  // DeviceManager::transferStaticPlaceholderToDevice (reference
  // include/glow/Backends/DeviceManager.h:166-171): copies `tensor` into the
  // device slot of the module's placeholder `placeholderName`. Requests that
  // do not bind that placeholder afterwards run on the transferred value (a
  // static placeholder: uploaded once, read by many requests). The module must
  // have a function resident on this device; a tensor larger than the slot, an
  // unknown name or a value that is no placeholder is a RUNTIME_ERROR.
  void transferStaticPlaceholderToDevice(const Module *module, std::string placeholderName,
                                         Tensor *tensor, std::function<void(Error)> resultCB);

  // Benchmark aid without a counterpart in the reference: replays a resident
  // function `iterations` times on the data its placeholders already hold (no
  // host copies) and reports the average device time per replay, measured
  // with events on the manager's stream. Blocks until done.
  Expected<float> timeFunction(const std::string &functionName, int iterations);

  uint64_t getMaximumMemory() const { return maxMemoryBytes_; }
  uint64_t getAvailableMemory() const { return maxMemoryBytes_ - usedMemoryBytes_; }
  bool isMemoryAvailable(uint64_t estimate) const {
    return maxMemoryBytes_ >= usedMemoryBytes_ + estimate;
  }
  DeviceInfo getDeviceInfo() const { return info_; }
  std::string getBackendName() const { return "MI355X"; }

private:
  struct ModuleResident {   // constants + placeholders of one module
    mi355x_arena *arena = nullptr;
    uint64_t bytes = 0;
    int users = 0;
  };
  struct FunctionResident {
    MI355XFunction *fn = nullptr;
    const Module *module = nullptr;
    mi355x_arena *arena = nullptr; // generated constants + activations
    uint64_t bytes = 0;
    DeviceBindings bindings;
    // branch tuning: requests 3c, 3c+1, 3c+2 go to candidate c (warm-up, timed, timed)
    std::vector<int> branchCandidates;
    std::vector<float> branchMs;
    int branchPhase = 0;
    bool branchesTuned = true;
  };

  void addNetworkImpl(const Module *module, FunctionMapTy functions, ReadyCBTy readyCB);
  void evictNetworkImpl(std::string functionName, EvictFunctionCBTy evictCB);
  void runFunctionImpl(RunIdentifierTy id, std::string functionName,
                       std::unique_ptr<ExecutionContext> ctx, ResultCBTy resultCB);
  Error makeResident(const Module *module, const std::string &name, MI355XFunction *fn);
  Error tuneTiles(MI355XFunction *fn, const DeviceBindings &b);
  Error captureWithBranches(FunctionResident &fr, int branches);
  Error executeTuned(FunctionResident &fr, ExecutionContext *ctx);
  void release(FunctionResident &fr);
  void enqueue(std::function<void()> work);
  int lengthsUploaded(const Module *module, const std::string &name, uint8_t *slot,
                      size_t slotBytes, const void *data, size_t bytes,
                      std::vector<std::vector<int32_t>> &staged);
  void workerLoop();

  DeviceConfig config_;
  DeviceInfo info_;
  std::atomic<uint64_t> maxMemoryBytes_{0}, usedMemoryBytes_{0};
  std::atomic<RunIdentifierTy> nextRun_{1};
  std::map<std::string, FunctionResident> functions_;
  std::map<const Module *, ModuleResident> modules_;
  void *stream_ = nullptr;
  std::vector<void *> sideStreams_; // branches of captured graphs

  std::thread worker_;
  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::function<void()>> queue_;
  bool running_ = false, stopping_ = false;
};

} // namespace glow_mi355x
#endif

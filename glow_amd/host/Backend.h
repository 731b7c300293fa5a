// MI355XBackend and MI355XFunction: the compile side of the drop-in boundary.
// Mirrors glow::Backend (reference include/glow/Backend/Backend.h:67-325) and
// glow::CompiledFunction (include/glow/Backend/CompiledFunction.h:29-98) for
// the quantized hot path; kernels are reached only through the C ABI of
// glow_mi355x.h.
#ifndef GLOW_MI355X_HOST_BACKEND_H
#define GLOW_MI355X_HOST_BACKEND_H

#include "Program.h"
#include "glow_mi355x.h"

#include <functional>
#include <map>
#include <memory>
#include <string>
#include <vector>

struct mi355x_graph;

namespace glow_mi355x {

// Where a run's buffers live on the device (ExecutionContext::DeviceBindings,
// reference include/glow/ExecutionContext/ExecutionContext.h:31-43).
struct DeviceBindings {
  uint8_t *constants = nullptr;   // module constants
  uint8_t *generated = nullptr;   // constants the compiler derived for one function
  uint8_t *mutableMem = nullptr;  // placeholders
  uint8_t *activations = nullptr; // one function's activations
  void *stream = nullptr;
  // Options every launch passes to the kernel library with the call itself
  // (the <entry>_opts forms): the device manager's SparseLengths arithmetic;
  // KernelLaunch::launch adds the launch's own tile and requantisation hint.
  mi355x_launch_opts opts = MI355X_LAUNCH_OPTS_INIT;
};

// PlaceholderBindings: placeholder name -> host tensor (not owned).
class PlaceholderBindings {
public:
  void insert(const std::string &name, Tensor *t) { map_[name] = t; }
  Tensor *get(const std::string &name) const {
    auto it = map_.find(name);
    return it == map_.end() ? nullptr : it->second;
  }
  const std::map<std::string, Tensor *> &pairs() const { return map_; }

private:
  std::map<std::string, Tensor *> map_;
};

class ExecutionContext {
public:
  PlaceholderBindings *getPlaceholderBindings() { return &bindings_; }
  void setDeviceBindings(std::unique_ptr<DeviceBindings> b) { device_ = std::move(b); }
  DeviceBindings *getDeviceBindings() { return device_.get(); }

private:
  PlaceholderBindings bindings_;
  std::unique_ptr<DeviceBindings> device_;
};

// RuntimeSymbolInfo (BackendUtils.h:41-62)
struct RuntimeSymbolInfo {
  size_t size = 0, offset = 0;
  Type type;
  bool input = false, output = false;
  SymbolCategory symbolCategory = SymbolCategory::Activation;
};

// RuntimeBundle (BackendUtils.h:66-150): sizes of the regions and the table.
struct RuntimeBundle {
  std::map<std::string, RuntimeSymbolInfo> symbolTable;
  size_t constantWeightVarsMemSize = 0;
  size_t mutableWeightVarsMemSize = 0;
  size_t activationsMemSize = 0;
  size_t generatedConstantsMemSize = 0; // no counterpart: kernel parameter vectors
  size_t getConstantWeightSize() const {
    return constantWeightVarsMemSize + generatedConstantsMemSize;
  }
};

// Memory a launch touches: the value (by its root, so views alias) and, for
// slices inserted into rows of a wider tensor, the byte range inside a row.
struct Access {
  int root = -1;
  long long lo = 0, hi = -1; // hi < 0: the whole value
  // activations only: the bytes [actLo, actHi) of the activations region the
  // root occupies (different values share memory when their lives do not meet)
  long long actLo = 0, actHi = 0;
  bool overlaps(const Access &o) const {
    if (root != o.root) return actLo < o.actHi && o.actLo < actHi;
    if (hi < 0 || o.hi < 0) return true;
    return lo < o.hi && o.lo < hi;
  }
};

// One kernel launch of a compiled function.
struct KernelLaunch {
  KernelLaunch(std::string k, std::string i, std::string p,
               std::function<int(const struct DeviceBindings &)> r)
      : kernel(std::move(k)), inst(std::move(i)), params(std::move(p)), run(std::move(r)) {}
  std::string kernel;  // C-ABI entry point
  std::string inst;    // instruction name
  std::string params;  // the derived integer parameters, for inspection
  std::function<int(const DeviceBindings &)> run; // returns an mi355x_status
  // Dependence information: launches of one level touch disjoint memory (or
  // only read common memory) and may run side by side.
  std::vector<Access> reads, writes;
  int level = 0;
  // Matrix-core launches can run with several workgroup tiles; `tile` is the
  // one to use (-1: the library's choice from the shape).
  bool tunable = false;
  int tile = -1;
  // Requantisation hint of a matrix-core launch (mi355x_gemm_requant_hint),
  // derived at compile time from the launch's constants with worst-case
  // operand bytes; 0 = none.
  int requantHint = 0;
  // Workspace of a matrix-core launch whose K loop the library may split over
  // workgroups (mi355x_gemm_splitk_workspace_bytes): workspaceBytes at
  // generated + *scratchBase + workspaceRel, its counters zeroed by a set-up
  // launch when the function is loaded; 0 bytes = none.
  size_t workspaceRel = 0, workspaceBytes = 0;
  std::shared_ptr<size_t> scratchBase;
  // Issues the launch (with its tile, hint and workspace, if it has them).
  int launch(const DeviceBindings &b) const;
};
constexpr int kNumTiles = 13;   // candidates -1 .. 12 of the tile tuner

class MI355XFunction {
public:
  MI355XFunction(RuntimeBundle bundle, std::string name)
      : bundle_(std::move(bundle)), name_(std::move(name)) {}
  ~MI355XFunction();

  // CompiledFunction::execute: the context must carry DeviceBindings (the
  // device manager sets them). Launches are asynchronous on the bound stream.
  Error execute(ExecutionContext *ctx);
  std::string getCompileBackendName() const { return "MI355X"; }
  const RuntimeBundle &getRuntimeBundle() const { return bundle_; }
  void setRuntimeBundle(RuntimeBundle b) { bundle_ = std::move(b); }
  const std::string &name() const { return name_; }

  // Launch lists: `setup` runs once after the constants are resident (weight
  // repacking, row sums); `launches` is the function body.
  std::vector<KernelLaunch> setup, launches;
  // Host image of the generated constants (uploaded by the device manager).
  std::vector<uint8_t> generated;
  // Where each value of the module lies in this function's activations region
  // (by value id; meaningful for the function's activations only). The launches
  // read it when they run.
  std::shared_ptr<std::vector<size_t>> activationOffsets;
  size_t activationsBytes = 0;   // size of the region so planned
  struct ActivationPlace {
    std::string name;
    int id;
    size_t offset, bytes;
  };
  std::vector<ActivationPlace> activationPlan;   // the values with memory of their own
  // Lookups whose lengths are an input placeholder read their bags as
  // positions: whoever uploads `lengths` also writes segments + 1 int32
  // exclusive prefix sums of the (clamped) lengths to ptr(bindings).
  struct DerivedBagOffsets {
    std::string lengths; // placeholder name
    size_t segments = 0;
    std::function<uint8_t *(const DeviceBindings &)> ptr;
  };
  std::vector<DerivedBagOffsets> derivedBagOffsets;
  // Placeholders (by name; a view counts for the value it views) that some
  // instruction of this function writes. Nobody may derive bag positions on
  // the host from such a placeholder: the device manager refuses to load two
  // functions of a module of which one writes what the other derives from.
  std::vector<std::string> writtenPlaceholders;
  // Host side of that contract: the positions for `lengths` (n of the
  // placeholder's `segments` entries given; the missing ones count as empty
  // bags). Sums saturate at INT32_MAX, which lies at or past the end of any
  // index list, where the kernels clamp positions anyway.
  static std::vector<int32_t> bagOffsets(const int32_t *lengths, size_t n, size_t segments);
  // Text listing of the launches with their parameters.
  std::string describe() const;

  // Records the body into a launch graph bound to these buffers; later
  // execute() calls with the same bindings replay it. With side streams the
  // launches of one dependence level are recorded as parallel branches.
  Error captureGraph(const DeviceBindings &b, const std::vector<void *> &sideStreams = {});
  void dropGraph();

private:
  RuntimeBundle bundle_;
  std::string name_;
  mi355x_graph *graph_ = nullptr;
  DeviceBindings graphBindings_;
};

struct BackendOptions {
  bool precomputeWeightRowSums = true; // form sum_k W[n][k] once at load time
  bool fuseAddRelu = true;             // ElementAdd + Relu of its result in one pass
  bool fuseConvAdd = true;             // convolution + ElementAdd (+ Relu) in one kernel
  bool spaceToDepthStem = true;        // stride-2 convolutions over <= 4 channels via space-to-depth
  bool fuseSlsChains = true;           // pooled lookups + ConvertTo/Quantize/InsertTensor, many tables per launch
  bool fuseTransposeMatMul = true;     // BatchMatMul(L, Transpose(R)) without materialising the transpose
  bool fuseFcRelu = true;              // RowwiseQuantizedFullyConnected + Relu of its result in one kernel
  bool padTableRows = true;            // constant lookup tables with 33..63-byte rows re-laid 64 bytes apart at load
  bool fuseInsert = true;              // Gather / RescaleQuantized write straight into the tensor their result is inserted into
  bool fuseDequantizeSigmoid = true;   // Dequantize + the Sigmoid or SoftMax of its result in one kernel
  bool deriveBagOffsets = true;        // lookups whose lengths are an input: bag positions summed on the host at upload
  bool fuseQuantizeStem = true;        // Quantize read only by a space-to-depth convolution: quantized while re-laid
  bool reuseActivations = true;        // activations whose lives do not meet share memory (first fit over the launch order)
  bool splitK = true;                  // matrix-core launches with few output tiles and a long K get a workspace, so the library may split K over workgroups
};

class MI355XBackend {
public:
  std::string getBackendName() const { return getName(); }
  static std::string getName() { return "MI355X"; }
  static unsigned numDevices(); // devices the runtime reports (0 without a GPU)

  // Backend::compile (Backend.h:108-109)
  Expected<std::unique_ptr<MI355XFunction>> compile(const Function &F,
                                                    const BackendOptions &opts = {}) const;
  // Backend::isOpSupported (Backend.h:145): by instruction kind and operand types.
  bool isOpSupported(const Module &M, const Instruction &I, std::string *why = nullptr) const;
  // Backend::shouldLower (Backend.h:197): FullyConnected, Convolution stay
  // un-lowered like on the CPU backend (CPUBackend.cpp:71-84).
  bool shouldLower(Kind k) const;
  // Backend::supportsFusedActivation (Backend.h:228-230, CPUBackend.cpp:86-112)
  bool supportsFusedActivation(Kind parent, FusedActivation act) const;
  // Backend::canDoIndexTypeDemotion: SLS indices stay int64 like on the CPU
  // backend (CPUBackend.cpp:147-159); int32 indices are accepted as given.
  bool canDoIndexTypeDemotion(Kind k) const { (void)k; return false; }
};

} // namespace glow_mi355x
#endif

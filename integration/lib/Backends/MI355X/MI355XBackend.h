/**
 * MI355X backend for Glow's quantized-inference path.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/Backend/Backend.h.
 */
#ifndef GLOW_BACKENDS_MI355X_MI355XBACKEND_H
#define GLOW_BACKENDS_MI355X_MI355XBACKEND_H

#include "glow/Backend/Backend.h"
#include "glow/Backend/BackendUtils.h"
#include "glow/Backends/DeviceManager.h"

#include <string>
#include <vector>

namespace glow {

class MI355XBackend final : public BackendUsingGlowIR {
public:
  MI355XBackend() = default;
  ~MI355XBackend() override = default;

  /// @name Backend methods.
  ///@{
  std::string getBackendName() const override {
    return Named::getName().empty() ? getName() : Named::getName().str();
  }
  static std::string getName() { return "MI355X"; }
  /// Number of gfx950 devices the HIP runtime reports (0 without one).
  static unsigned numDevices();
  static std::vector<unsigned> scanDeviceIDs();

  Expected<std::unique_ptr<CompiledFunction>>
  compile(Function *F, const BackendOptions &opts) const override;

  std::unique_ptr<CompiledFunction>
  compileIR(std::unique_ptr<IRFunction> IR) const override;

  /// The quantized subset of lib/LLVMIRCodeGen/LLVMBackend.cpp:52-584 plus the
  /// data-movement nodes a quantized ResNet / ranking model needs.
  bool isOpSupported(const NodeInfo &NI) const override;

  /// FullyConnected, Convolution, Relu and Clip stay un-lowered, as on the CPU
  /// backend (lib/Backends/CPU/CPUBackend.cpp:71-84): each has a kernel of its
  /// own here.
  bool shouldLower(const Node *N) const override;

  /// Relu / Clip / LeakyRelu into Convolution and
  /// ChannelwiseQuantizedConvolution (CPUBackend.cpp:86-112); quantized
  /// Sigmoid / Tanh are not fused (they become lookup tables upstream).
  bool supportsFusedActivation(Node *parent, Node *activation) const override;

  /// Nothing is rewritten at the graph level: every fusion of this backend is
  /// a peephole over the lowered instruction list (MI355XFunction), which sees
  /// the final buffers and their single readers.
  Expected<bool> transformPostLowering(
      Function *F, CompilationContext &cctx,
      const glow::runtime::DeviceInfo *devInfo = nullptr) const override;

  /// int64 -> int32 index demotion everywhere except the SparseLengths family
  /// (the kernels take either; the reference keeps them int64 on the CPU,
  /// CPUBackend.cpp:147-159, and so the same graphs arrive here).
  bool canDoIndexTypeDemotion(ElemKind fromTy, ElemKind toTy,
                              PrecisionConfiguration &precConfig) const override;

  /// The IR optimizer's buffer sharing is wanted: fewer, larger activations.
  bool shouldShareBuffers() const override { return true; }

  /// Index tensors are statically sized and only partly used per request.
  bool supportsPartialTensors() const override { return true; }
  bool supportsStaticPlaceholders() const override { return true; }

  runtime::DeviceManager *
  createDeviceManager(const runtime::DeviceConfig &deviceConfig) override;
  ///@}
};

} // namespace glow

#endif // GLOW_BACKENDS_MI355X_MI355XBACKEND_H

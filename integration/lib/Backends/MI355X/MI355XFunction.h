/**
 * MI355XFunction: a Glow IRFunction compiled into MI355X kernel launches.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/Backend/CompiledFunction.h and
 * include/glow/IR/IR.h.
 */
#ifndef GLOW_BACKENDS_MI355X_MI355XFUNCTION_H
#define GLOW_BACKENDS_MI355X_MI355XFUNCTION_H

#include "glow/Backend/BackendOptions.h"
#include "glow/Backend/CompiledFunction.h"
#include "glow/ExecutionContext/ExecutionContext.h"
#include "glow/Graph/Graph.h"
#include "glow/IR/IR.h"

// the MI355X host layer (glow_amd/host in the kernel library's repository)
#include "Backend.h"
#include "Program.h"

#include <memory>
#include <string>
#include <unordered_map>

namespace glow {

/// What the device manager puts into the ExecutionContext before
/// CompiledFunction::execute: where the function's regions live on the device
/// and the stream to launch on (the OpenCL backend's pattern,
/// lib/Backends/OpenCL/OpenCLDeviceManager.cpp:775-845).
class MI355XDeviceBindings final : public DeviceBindings {
public:
  explicit MI355XDeviceBindings(const glow_mi355x::DeviceBindings &b)
      : DeviceBindings("MI355X"), device(b) {}
  std::unique_ptr<DeviceBindings> clone() override {
    return glow::make_unique<MI355XDeviceBindings>(device);
  }
  glow_mi355x::DeviceBindings device;
};

class MI355XFunction final : public CompiledFunction {
public:
  explicit MI355XFunction(runtime::RuntimeBundle &&bundle);
  ~MI355XFunction() override;

  /// Restates \p IR for the host layer (same instruction names, same operand
  /// order) and compiles it into kernel launches. Constants are copied out of
  /// \p mod here: the Module may be stripped after deployment.
  Error build(const IRFunction &IR, const Module &mod,
              const BackendOptions &opts);

  /// @name CompiledFunction interface
  ///@{
  Error execute(ExecutionContext *context) override;
  void collectConstants(const Module *module) override;
  std::string getCompileBackendName() const override { return "MI355X"; }
  /// The host copies of the constants are not needed once the device manager
  /// has uploaded them.
  void freeCompilationResources() override;
  const std::string toJSON() const override;
  ///@}

  /// The compiled launch lists and the module they were compiled from; the
  /// device manager makes both resident.
  glow_mi355x::MI355XFunction *hostFunction() { return compiled_.get(); }
  const glow_mi355x::Module *hostModule() const { return hostModule_.get(); }

private:
  std::unique_ptr<glow_mi355x::Module> hostModule_;
  std::unique_ptr<glow_mi355x::MI355XFunction> compiled_;
};

/// glow_mi355x::Error -> glow::Error with the same code.
Error toGlowError(const glow_mi355x::Error &e);

} // namespace glow

#endif // GLOW_BACKENDS_MI355X_MI355XFUNCTION_H

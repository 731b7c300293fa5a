/**
 * MI355XFunction: restates a Glow IRFunction for the MI355X host layer and
 * runs the launches it compiles to.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/IR/IR.h, include/glow/IR/Instrs.h
 * (generated from tools/ClassGen/InstrGen.cpp) and include/glow/IR/IRUtils.h.
 */
#include "MI355XFunction.h"

#include "glow/IR/IRUtils.h"
#include "glow/IR/Instrs.h"
#include "glow/Support/Error.h"

#include "llvm/Support/Casting.h"

using namespace glow;
using llvm::cast;
using llvm::dyn_cast;

namespace hm = glow_mi355x;

Error glow::toGlowError(const hm::Error &e) {
  if (!e) {
    return Error::success();
  }
  using EC = ErrorValue::ErrorCode;
  EC code = EC::RUNTIME_ERROR;
  switch (e.code()) {
  case hm::ErrorCode::RUNTIME_OUT_OF_DEVICE_MEMORY:
    code = EC::RUNTIME_OUT_OF_DEVICE_MEMORY;
    break;
  case hm::ErrorCode::RUNTIME_NET_NOT_FOUND:
    code = EC::RUNTIME_NET_NOT_FOUND;
    break;
  case hm::ErrorCode::RUNTIME_REQUEST_REFUSED:
    code = EC::RUNTIME_REQUEST_REFUSED;
    break;
  case hm::ErrorCode::RUNTIME_DEVICE_NOT_FOUND:
    code = EC::RUNTIME_DEVICE_NOT_FOUND;
    break;
  case hm::ErrorCode::RUNTIME_DEVICE_NONRECOVERABLE:
    code = EC::RUNTIME_DEVICE_NONRECOVERABLE;
    break;
  case hm::ErrorCode::RUNTIME_NET_BUSY:
    code = EC::RUNTIME_NET_BUSY;
    break;
  case hm::ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED:
    code = EC::DEVICE_FEATURE_NOT_SUPPORTED;
    break;
  case hm::ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE:
    code = EC::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE;
    break;
  case hm::ErrorCode::COMPILE_CONTEXT_MALFORMED:
    code = EC::COMPILE_CONTEXT_MALFORMED;
    break;
  default:
    break;
  }
  return MAKE_ERR(code, e.message());
}

/// glow::Type -> the host layer's type. \returns false for an element kind the
/// path does not carry.
static bool toHostType(const Type &t, hm::Type &out) {
  hm::ElemKind k;
  switch (t.getElementType()) {
  case ElemKind::FloatTy:
    k = hm::ElemKind::FloatTy;
    break;
  case ElemKind::Float16Ty:
    k = hm::ElemKind::Float16Ty;
    break;
  case ElemKind::Int8QTy:
  case ElemKind::UInt8QTy: // rowwise (not fused) lookup tables: raw bytes
    k = hm::ElemKind::Int8QTy;
    break;
  case ElemKind::Int32QTy:
    k = hm::ElemKind::Int32QTy;
    break;
  case ElemKind::Int16QTy:
    k = hm::ElemKind::Int16QTy;
    break;
  case ElemKind::Int32ITy:
    k = hm::ElemKind::Int32ITy;
    break;
  case ElemKind::Int64ITy:
    k = hm::ElemKind::Int64ITy;
    break;
  case ElemKind::UInt8FusedQTy:
    k = hm::ElemKind::UInt8FusedQTy;
    break;
  case ElemKind::UInt8FusedFP16QTy:
    k = hm::ElemKind::UInt8FusedFP16QTy;
    break;
  case ElemKind::UInt4FusedFP16QTy:
    k = hm::ElemKind::UInt4FusedFP16QTy;
    break;
  case ElemKind::UInt4FusedQTy:
    k = hm::ElemKind::UInt4FusedQTy;
    break;
  case ElemKind::BoolTy:
    k = hm::ElemKind::BoolTy;
    break;
  default:
    return false;
  }
  std::vector<int64_t> dims(t.dims().begin(), t.dims().end());
  if (t.isQuantizedType() && !t.isFusedQuantizedType()) {
    out = hm::Type(k, std::move(dims), t.getScale(), t.getOffset());
  } else {
    out = hm::Type(k, std::move(dims));
  }
  return true;
}

namespace {

/// Builds the host layer's Module / Function from one IRFunction.
class Translator {
public:
  Translator(const IRFunction &IR, const Module &mod, hm::Module &out)
      : IR_(IR), mod_(mod), out_(out) {}

  Error run(hm::Function *&fnOut) {
    RETURN_IF_ERR(weights());
    fn_ = out_.createFunction(IR_.getName().str());
    for (const auto &I : IR_.getInstrs()) {
      RETURN_IF_ERR(instruction(I));
    }
    fnOut = fn_;
    return Error::success();
  }

private:
  const IRFunction &IR_;
  const Module &mod_;
  hm::Module &out_;
  hm::Function *fn_ = nullptr;
  std::unordered_map<const Value *, int> ids_;

  Error unsupported(const Instruction &I, const std::string &why) {
    return MAKE_ERR(ErrorValue::ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE,
                    strFormat("MI355X: %s '%s': %s", I.getKindName(),
                              I.getName().str().c_str(), why.c_str()));
  }

  /// Constants (payload copied) and Placeholders of the function, under the
  /// names the RuntimeBundle's symbol table uses.
  Error weights() {
    for (const auto &kv : IR_.getVariableMap()) {
      const Storage *S = kv.first;
      const Value *W = kv.second;
      hm::Type ty;
      if (!toHostType(*W->getType(), ty)) {
        return MAKE_ERR(
            ErrorValue::ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE,
            strFormat("MI355X: weight '%s' has element kind %s",
                      W->getName().str().c_str(),
                      Type::getElementName(W->getElementType()).str().c_str()));
      }
      int id = -1;
      if (const auto *C = dyn_cast<Constant>(S)) {
        id = out_.createConstant(W->getName().str(), ty,
                                 C->getPayload().getUnsafePtr());
      } else {
        id = out_.createPlaceholder(W->getName().str(), ty);
      }
      ids_[W] = id;
    }
    (void)mod_;
    return Error::success();
  }

  Expected<int> idOf(const Instruction &I, const Value *V) {
    auto it = ids_.find(V);
    if (it == ids_.end()) {
      return unsupported(I, strFormat("operand '%s' was not allocated before use",
                                      V->getName().str().c_str()));
    }
    return it->second;
  }

  /// The operands of \p I in IR order (Dest first), which is the host layer's
  /// order for every kind below.
  Expected<std::vector<int>> operandIds(const Instruction &I) {
    std::vector<int> r;
    for (unsigned i = 0, e = I.getNumOperands(); i < e; i++) {
      int id;
      ASSIGN_VALUE_OR_RETURN_ERR(id, idOf(I, I.getOperand(i).first));
      r.push_back(id);
    }
    return r;
  }

  template <class ConvInst>
  hm::ConvAttrs convAttrs(const ConvInst *C) {
    hm::ConvAttrs a;
    a.kernelH = C->getKernels()[0];
    a.kernelW = C->getKernels()[1];
    a.strideH = C->getStrides()[0];
    a.strideW = C->getStrides()[1];
    a.padT = C->getPads()[0]; // Glow's order is top, left, bottom, right
    a.padL = C->getPads()[1];
    a.padB = C->getPads()[2];
    a.padR = C->getPads()[3];
    a.group = C->getGroup();
    a.dilationH = C->getDilation()[0];
    a.dilationW = C->getDilation()[1];
    a.fusedActivation = static_cast<int64_t>(C->getFusedActivation());
    return a;
  }

  static std::vector<int64_t> poolAttrs(llvm::ArrayRef<unsigned_t> k,
                                        llvm::ArrayRef<unsigned_t> s,
                                        llvm::ArrayRef<unsigned_t> p) {
    return {k[0], k[1], s[0], s[1], p[0], p[1], p[2], p[3]};
  }

  Error add(const Instruction &I, hm::Kind kind, std::vector<int64_t> iattrs = {},
            std::vector<float> fattrs = {}) {
    std::vector<int> ops;
    ASSIGN_VALUE_OR_RETURN_ERR(ops, operandIds(I));
    fn_->addInstruction(kind, I.getName().str(), std::move(ops), std::move(iattrs),
                        std::move(fattrs));
    return Error::success();
  }

  Error instruction(const Instruction &I) {
    switch (I.getKind()) {
    // ---- memory ------------------------------------------------------------
    case Kinded::Kind::AllocActivationInstKind: {
      hm::Type ty;
      if (!toHostType(*I.getType(), ty)) {
        return unsupported(I, "element kind not carried by this backend");
      }
      ids_[&I] = fn_->createActivation(I.getName().str(), ty);
      return Error::success();
    }
    case Kinded::Kind::DeallocActivationInstKind:
    case Kinded::Kind::TouchInstKind:
      return Error::success();
    case Kinded::Kind::TensorViewInstKind: {
      const auto *TV = cast<TensorViewInst>(&I);
      // a reshape of the buffer, or a slice of the outermost dimension of a
      // placeholder or constant (the bytes stay contiguous): the flat offset of
      // Tensor::getUnowned(ty, offsets) for offsets = {o, 0, 0, ...}
      size_t byteOffset = 0;
      const auto offs = TV->getOffsets();
      for (size_t k = 1; k < offs.size(); k++) {
        if (offs[k] != 0) {
          return unsupported(I, "tensor views with inner offsets are not supported");
        }
      }
      if (!offs.empty() && offs[0] != 0) {
        const TypeRef srcTy = TV->getSrc()->getType();
        byteOffset = (size_t)offs[0] * (srcTy->size() / srcTy->dims()[0]) *
                     srcTy->getElementSize();
      }
      hm::Type ty;
      if (!toHostType(*TV->getTy(), ty)) {
        return unsupported(I, "element kind not carried by this backend");
      }
      int src;
      ASSIGN_VALUE_OR_RETURN_ERR(src, idOf(I, TV->getSrc()));
      const int id = out_.createView(I.getName().str(), src, ty, byteOffset);
      if (id < 0) {
        return unsupported(I, "view outside its source, or a slice of an activation");
      }
      ids_[&I] = id;
      return Error::success();
    }
    case Kinded::Kind::CopyInstKind:
      return add(I, hm::Kind::Copy);

    // ---- the quantization boundary ------------------------------------------
    case Kinded::Kind::QuantizeInstKind:
      return add(I, hm::Kind::Quantize);
    case Kinded::Kind::DequantizeInstKind:
      return add(I, hm::Kind::Dequantize);
    case Kinded::Kind::RescaleQuantizedInstKind:
      return add(I, hm::Kind::RescaleQuantized);

    // ---- matrix-core operators ------------------------------------------------
    case Kinded::Kind::FullyConnectedInstKind:
      return add(I, hm::Kind::FullyConnected);
    case Kinded::Kind::RowwiseQuantizedFullyConnectedInstKind:
      return add(I, hm::Kind::RowwiseQuantizedFullyConnected);
    case Kinded::Kind::MatMulInstKind:
      return add(I, hm::Kind::MatMul);
    case Kinded::Kind::BatchMatMulInstKind:
      return add(I, hm::Kind::BatchMatMul);
    case Kinded::Kind::ConvolutionInstKind: {
      const auto *C = cast<ConvolutionInst>(&I);
      if (C->getLayout() != NHWC) {
        return unsupported(I, "only NHWC convolutions are supported");
      }
      const hm::ConvAttrs a = convAttrs(C);
      std::vector<int> ops;
      ASSIGN_VALUE_OR_RETURN_ERR(ops, operandIds(I));
      fn_->createConvolution(I.getName().str(), ops[0], ops[1], ops[2], ops[3], a,
                             C->getFusedActivationArgs());
      return Error::success();
    }
    case Kinded::Kind::ChannelwiseQuantizedConvolutionInstKind: {
      const auto *C = cast<ChannelwiseQuantizedConvolutionInst>(&I);
      if (C->getSrc()->dims().size() == 5) {
        // NTHWC: kernels {T,H,W}, strides {T,H,W}, pads {near, far, top, bottom,
        // left, right} (PaddingNFTBLR), group, fused activation, in the order
        // the host layer's 3-D form takes its integer attributes
        std::vector<int64_t> ia;
        for (auto v : C->getKernels()) ia.push_back((int64_t)v);
        for (auto v : C->getStrides()) ia.push_back((int64_t)v);
        for (auto v : C->getPads()) ia.push_back((int64_t)v);
        if (ia.size() != 12) {
          return unsupported(I, "a 3-D convolution needs 3 kernels, 3 strides and 6 pads");
        }
        for (auto d : C->getDilation()) {
          if (d != 1) return unsupported(I, "dilated 3-D convolutions are not supported");
        }
        ia.push_back((int64_t)C->getGroup());
        ia.push_back((int64_t)C->getFusedActivation());
        std::vector<int> ops;
        ASSIGN_VALUE_OR_RETURN_ERR(ops, operandIds(I));
        fn_->addInstruction(hm::Kind::ChannelwiseQuantizedConvolution, I.getName().str(), ops,
                            std::move(ia), C->getFusedActivationArgs());
        return Error::success();
      }
      if (C->getSrc()->dims().size() != 4) {
        return unsupported(I, "needs an NHWC or NTHWC input");
      }
      const hm::ConvAttrs a = convAttrs(C);
      std::vector<int> ops;
      ASSIGN_VALUE_OR_RETURN_ERR(ops, operandIds(I));
      fn_->createChannelwiseQuantizedConvolution(
          I.getName().str(), ops[0], ops[1], ops[2], ops[3], ops[4], ops[5], ops[6],
          ops[7], a, C->getFusedActivationArgs());
      return Error::success();
    }

    // ---- pooled lookups ----------------------------------------------------------
    case Kinded::Kind::FusedRowwiseQuantizedSparseLengthsWeightedSumInstKind: {
      const auto *S = cast<FusedRowwiseQuantizedSparseLengthsWeightedSumInst>(&I);
      return add(I, hm::Kind::FusedRowwiseQuantizedSparseLengthsWeightedSum,
                 {S->getUseFP16Accumulation() ? 1 : 0});
    }
    case Kinded::Kind::FusedRowwiseQuantizedSparseLengthsSumInstKind: {
      const auto *S = cast<FusedRowwiseQuantizedSparseLengthsSumInst>(&I);
      return add(I, hm::Kind::FusedRowwiseQuantizedSparseLengthsSum,
                 {S->getUseFP16Accumulation() ? 1 : 0});
    }
    case Kinded::Kind::RowwiseQuantizedSparseLengthsWeightedSumInstKind:
      return add(I, hm::Kind::RowwiseQuantizedSparseLengthsWeightedSum);
    case Kinded::Kind::EmbeddingBagByteRowwiseOffsetsInstKind: {
      const auto *E = cast<EmbeddingBagByteRowwiseOffsetsInst>(&I);
      return add(I, hm::Kind::EmbeddingBagByteRowwiseOffsets,
                 {E->getHasEndOffset() ? 1 : 0});
    }

    // ---- int8 glue -----------------------------------------------------------------
    case Kinded::Kind::ElementAddInstKind:
      return add(I, hm::Kind::ElementAdd);
    case Kinded::Kind::ReluInstKind:
      return add(I, hm::Kind::Relu);
    case Kinded::Kind::ClipInstKind: {
      const auto *C = cast<ClipInst>(&I);
      return add(I, hm::Kind::Clip, {}, {C->getMin(), C->getMax()});
    }
    case Kinded::Kind::LeakyReluInstKind: {
      const auto *L = cast<LeakyReluInst>(&I);
      return add(I, hm::Kind::LeakyRelu, {}, {L->getAlpha()});
    }
    case Kinded::Kind::BatchedAddInstKind:
      return add(I, hm::Kind::BatchedAdd);
#ifdef GLOW_WITH_CPU
    case Kinded::Kind::CPUMaxSplatInstKind: {
      const auto *S = cast<CPUMaxSplatInst>(&I);
      return add(I, hm::Kind::CPUMaxSplat, {}, {S->getSplatValue()});
    }
#endif
    case Kinded::Kind::MaxPoolInstKind: {
      const auto *P = cast<MaxPoolInst>(&I);
      if (P->getLayout() != NHWC) {
        return unsupported(I, "only NHWC pooling is supported");
      }
      return add(I, hm::Kind::MaxPool,
                 poolAttrs(P->getKernels(), P->getStrides(), P->getPads()));
    }
    case Kinded::Kind::AvgPoolInstKind: {
      const auto *P = cast<AvgPoolInst>(&I);
      if (P->getLayout() != NHWC) {
        return unsupported(I, "only NHWC pooling is supported");
      }
      auto a = poolAttrs(P->getKernels(), P->getStrides(), P->getPads());
      a.push_back(P->getCountIncludePads() ? 1 : 0);
      return add(I, hm::Kind::AvgPool, std::move(a));
    }
    case Kinded::Kind::SoftMaxInstKind:
      return add(I, hm::Kind::SoftMax);
    case Kinded::Kind::SigmoidInstKind:
      return add(I, hm::Kind::Sigmoid);

    // ---- data movement ---------------------------------------------------------------
    case Kinded::Kind::ConvertToInstKind:
      return add(I, hm::Kind::ConvertTo);
    case Kinded::Kind::InsertTensorInstKind: {
      const auto *T = cast<InsertTensorInst>(&I);
      // rows of a 2-D tensor, inserted once along the inner dimension
      if (T->getCount() != 1 || T->getOffsets().size() != 2 || T->getOffsets()[0] != 0) {
        return unsupported(I, "only a single insertion at {0, offset} into a 2-D "
                              "tensor is supported");
      }
      return add(I, hm::Kind::InsertTensor, {(int64_t)T->getOffsets()[1]});
    }
    case Kinded::Kind::TransposeInstKind: {
      const auto *T = cast<TransposeInst>(&I);
      std::vector<int64_t> shuffle(T->getShuffle().begin(), T->getShuffle().end());
      return add(I, hm::Kind::Transpose, std::move(shuffle));
    }
    case Kinded::Kind::GatherInstKind: {
      const auto *G = cast<GatherInst>(&I);
      return add(I, hm::Kind::Gather, {(int64_t)G->getBatchDims()});
    }

    default:
      return unsupported(I, "no MI355X kernel for this instruction");
    }
  }
};

} // namespace

MI355XFunction::MI355XFunction(runtime::RuntimeBundle &&bundle)
    : CompiledFunction(std::move(bundle)) {}

MI355XFunction::~MI355XFunction() = default;

Error MI355XFunction::build(const IRFunction &IR, const Module &mod,
                            const BackendOptions &opts) {
  hostModule_ = glow::make_unique<hm::Module>(mod.getName().str());
  hm::Function *fn = nullptr;
  RETURN_IF_ERR(Translator(IR, mod, *hostModule_).run(fn));

  // Backend-specific options: "MI355X_<name>" = 0 switches a peephole off
  // (all are on by default; see glow_mi355x::BackendOptions).
  hm::BackendOptions ho;
  auto off = [&](const char *key) {
    auto it = opts.backendSpecificOpts.find(std::string("MI355X_") + key);
    return it != opts.backendSpecificOpts.end() && it->second == "0";
  };
  if (off("fuseAddRelu")) ho.fuseAddRelu = false;
  if (off("fuseConvAdd")) ho.fuseConvAdd = false;
  if (off("spaceToDepthStem")) ho.spaceToDepthStem = false;
  if (off("fuseSlsChains")) ho.fuseSlsChains = false;
  if (off("fuseTransposeMatMul")) ho.fuseTransposeMatMul = false;
  if (off("fuseFcRelu")) ho.fuseFcRelu = false;
  if (off("padTableRows")) ho.padTableRows = false;
  if (off("fuseInsert")) ho.fuseInsert = false;
  if (off("fuseDequantizeSigmoid")) ho.fuseDequantizeSigmoid = false;
  if (off("precomputeWeightRowSums")) ho.precomputeWeightRowSums = false;
  if (off("deriveBagOffsets")) ho.deriveBagOffsets = false;
  if (off("reuseActivations")) ho.reuseActivations = false;
  if (off("fuseQuantizeStem")) ho.fuseQuantizeStem = false;

  hm::MI355XBackend hostBackend;
  auto compiled = hostBackend.compile(*fn, ho);
  if (!compiled) {
    return toGlowError(compiled.error());
  }
  compiled_ = std::move(compiled.get());
  return Error::success();
}

void MI355XFunction::collectConstants(const Module *module) {
  // Glow-side bundle bookkeeping (sizes for DeviceManager accounting); the
  // payloads the device needs were copied in build().
  runtimeBundle_.collectConstants(module);
}

void MI355XFunction::freeCompilationResources() {
  runtimeBundle_.freeConstants();
}

const std::string MI355XFunction::toJSON() const {
  // not JSON proper: the launch listing with every derived integer parameter
  return compiled_ ? compiled_->describe() : std::string();
}

Error MI355XFunction::execute(ExecutionContext *context) {
  // DeviceBindings carries no RTTI of its own; the device manager of this
  // backend is the only one that hands a context to this function (the OpenCL
  // backend does the same cast, lib/Backends/OpenCL/OpenCL.cpp)
  auto *bindings =
      static_cast<MI355XDeviceBindings *>(context->getDeviceBindings());
  if (!bindings || !compiled_) {
    return MAKE_ERR(ErrorValue::ErrorCode::RUNTIME_ERROR,
                    "MI355XFunction::execute needs device bindings from "
                    "MI355XDeviceManager");
  }
  hm::ExecutionContext hostCtx;
  hostCtx.setDeviceBindings(
      std::unique_ptr<hm::DeviceBindings>(new hm::DeviceBindings(bindings->device)));
  return toGlowError(compiled_->execute(&hostCtx));
}

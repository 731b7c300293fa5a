/**
 * MI355X backend for Glow's quantized-inference path: the Backend side.
 *
 * NOT COMPILED in the repository this file ships in (no LLVM/glog/folly
 * there); written against include/glow/Backend/Backend.h,
 * include/glow/Graph/Nodes.h and include/glow/Optimizer/IROptimizer.
 */
#include "MI355XBackend.h"
#include "MI355XDeviceManager.h"
#include "MI355XFunction.h"

#include "glow/Backend/BackendUtils.h"
#include "glow/Graph/Graph.h"
#include "glow/Graph/Nodes.h"
#include "glow/IR/IR.h"
#include "glow/IR/Instrs.h"
#include "glow/Optimizer/IROptimizer/IROptimizer.h"
#include "glow/Support/Memory.h"

#include "glow_mi355x.h" // mi355x_num_devices

#include <numeric>

using namespace glow;

unsigned MI355XBackend::numDevices() {
  int n = 0;
  if (mi355x_num_devices(&n) != MI355X_OK || n < 0) {
    return 0;
  }
  return static_cast<unsigned>(n);
}

std::vector<unsigned> MI355XBackend::scanDeviceIDs() {
  std::vector<unsigned> ids(MI355XBackend::numDevices());
  std::iota(ids.begin(), ids.end(), 0);
  return ids;
}

Expected<std::unique_ptr<CompiledFunction>>
MI355XBackend::compile(Function *F, const BackendOptions &opts) const {
  TraceInfo traceInfo = buildManualTraceInfo(F);
  auto IR = generateAndOptimizeIR(F, *this, shouldShareBuffers());
  if (opts.autoInstrument) {
    autoInstrument(traceInfo, IR.get());
  }
  const Module *mod = IR->getParent();
  MemoryAllocator constantWeightsAllocator("ConstantWeights", 0);
  MemoryAllocator placeholderWeightsAllocator("PlaceholderWeights", 0);
  MemoryAllocator activationsAllocator("Activations", 0);
  runtime::RuntimeBundle bundle = runtime::RuntimeBundle::create(
      *IR, constantWeightsAllocator, placeholderWeightsAllocator,
      activationsAllocator);
  auto function = glow::make_unique<MI355XFunction>(std::move(bundle));
  // The instruction stream is restated for the host layer and compiled into
  // kernel launches here, while the Module (and its constants) is still whole:
  // Backend::shouldStripModule() lets the runtime drop payloads afterwards.
  RETURN_IF_ERR(function->build(*IR, *mod, opts));
  if (opts.collectConstants) {
    function->collectConstants(mod);
  }
  function->setTraceInfo(std::move(traceInfo));
  return Expected<std::unique_ptr<CompiledFunction>>(std::move(function));
}

std::unique_ptr<CompiledFunction>
MI355XBackend::compileIR(std::unique_ptr<IRFunction> IR) const {
  const Module *mod = IR->getParent();
  MemoryAllocator constantWeightsAllocator("ConstantWeights", 0);
  MemoryAllocator placeholderWeightsAllocator("PlaceholderWeights", 0);
  MemoryAllocator activationsAllocator("Activations", 0);
  runtime::RuntimeBundle bundle = runtime::RuntimeBundle::create(
      *IR, constantWeightsAllocator, placeholderWeightsAllocator,
      activationsAllocator);
  auto function = glow::make_unique<MI355XFunction>(std::move(bundle));
  BackendOptions opts;
  // unit tests that hand IR in cannot receive an Error: an instruction this
  // backend does not know is fatal here, as it is in the Interpreter
  EXIT_ON_ERR(function->build(*IR, *mod, opts));
  function->collectConstants(mod);
  return function;
}

/// \returns true when the index operand \p idx of \p NI is int32 or int64.
static bool indexIs32or64(const NodeInfo &NI, unsigned idx) {
  return NI.getInElemTy(idx) == ElemKind::Int32ITy ||
         NI.getInElemTy(idx) == ElemKind::Int64ITy;
}

/// The fused-rowwise lookups accept what the reference's Interpreter accepts
/// (lib/Backends/Interpreter/Interpreter.cpp:526-567): fp32-scale tables with
/// (float weights, float result) or (fp16, fp16); fp16-scale tables with a
/// Float16 result and float or fp16 weights.
static bool fusedLookupTypesOk(ElemKind data, bool hasWeights, ElemKind weights,
                               ElemKind result) {
  switch (data) {
  case ElemKind::UInt8FusedQTy:
  case ElemKind::UInt4FusedQTy:
    if (result == ElemKind::FloatTy) {
      return !hasWeights || weights == ElemKind::FloatTy;
    }
    return result == ElemKind::Float16Ty &&
           (!hasWeights || weights == ElemKind::Float16Ty);
  case ElemKind::UInt8FusedFP16QTy:
  case ElemKind::UInt4FusedFP16QTy:
    return result == ElemKind::Float16Ty &&
           (!hasWeights || weights == ElemKind::FloatTy ||
            weights == ElemKind::Float16Ty);
  default:
    return false;
  }
}

static bool isQuantizedIntKind(ElemKind k) {
  return k == ElemKind::Int8QTy || k == ElemKind::Int16QTy || k == ElemKind::Int32QTy;
}

bool MI355XBackend::isOpSupported(const NodeInfo &NI) const {
  // "X ==> Y" below: Node X is IRGen'd into Instruction Y.
  switch (NI.getKind()) {

  // ---- the quantization boundary -----------------------------------------
  // (int8 is the hot path; the 16- and 32-bit forms of
  // libjit.cpp:3004-3056 run as plain elementwise kernels)
  case Kinded::Kind::QuantizeNodeKind:
    return NI.getInElemTy(QuantizeNode::InputIdx) == ElemKind::FloatTy &&
           isQuantizedIntKind(NI.getOutElemTy(QuantizeNode::ResultIdx));

  case Kinded::Kind::DequantizeNodeKind:
    return isQuantizedIntKind(NI.getInElemTy(DequantizeNode::InputIdx)) &&
           NI.getOutElemTy(DequantizeNode::ResultIdx) == ElemKind::FloatTy;

  case Kinded::Kind::RescaleQuantizedNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind(
        {ElemKind::Int8QTy, ElemKind::Int16QTy, ElemKind::Int32QTy});

  // ---- matrix-core operators ---------------------------------------------
  case Kinded::Kind::FullyConnectedNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind(
               {ElemKind::Int8QTy}, {FullyConnectedNode::BiasIdx}) &&
           (NI.getInElemTy(FullyConnectedNode::BiasIdx) == ElemKind::Int8QTy ||
            NI.getInElemTy(FullyConnectedNode::BiasIdx) == ElemKind::Int32QTy);

  case Kinded::Kind::RowwiseQuantizedFullyConnectedNodeKind:
    return NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::InputIdx) ==
               ElemKind::Int8QTy &&
           NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::WeightsIdx) ==
               ElemKind::Int8QTy &&
           NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::ScalesIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::OffsetsIdx) ==
               ElemKind::Int32ITy &&
           (NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::BiasIdx) ==
                ElemKind::Int8QTy ||
            NI.getInElemTy(RowwiseQuantizedFullyConnectedNode::BiasIdx) ==
                ElemKind::Int32QTy) &&
           NI.getOutElemTy(RowwiseQuantizedFullyConnectedNode::ResultIdx) ==
               ElemKind::Int8QTy;

  case Kinded::Kind::MatMulNodeKind:
  case Kinded::Kind::BatchMatMulNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy});

  case Kinded::Kind::ConvolutionNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy},
                                                  {ConvolutionNode::BiasIdx}) &&
           (NI.getInElemTy(ConvolutionNode::BiasIdx) == ElemKind::Int8QTy ||
            NI.getInElemTy(ConvolutionNode::BiasIdx) == ElemKind::Int32QTy);

  case Kinded::Kind::ChannelwiseQuantizedConvolutionNodeKind:
    return NI.getInElemTy(ChannelwiseQuantizedConvolutionNode::InputIdx) ==
               ElemKind::Int8QTy &&
           NI.getInElemTy(ChannelwiseQuantizedConvolutionNode::FilterIdx) ==
               ElemKind::Int8QTy &&
           (NI.getInElemTy(ChannelwiseQuantizedConvolutionNode::BiasIdx) ==
                ElemKind::Int8QTy ||
            NI.getInElemTy(ChannelwiseQuantizedConvolutionNode::BiasIdx) ==
                ElemKind::Int32QTy) &&
           NI.getInElemTy(
               ChannelwiseQuantizedConvolutionNode::FilterScalesIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(
               ChannelwiseQuantizedConvolutionNode::FilterOffsetsIdx) ==
               ElemKind::Int32ITy &&
           NI.getInElemTy(ChannelwiseQuantizedConvolutionNode::BiasScalesIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(
               ChannelwiseQuantizedConvolutionNode::BiasOffsetsIdx) ==
               ElemKind::Int32ITy &&
           NI.getOutElemTy(ChannelwiseQuantizedConvolutionNode::ResultIdx) ==
               ElemKind::Int8QTy;

  // ---- pooled lookups ------------------------------------------------------
  case Kinded::Kind::FusedRowwiseQuantizedSparseLengthsWeightedSumNodeKind:
    return fusedLookupTypesOk(
               NI.getInElemTy(
                   FusedRowwiseQuantizedSparseLengthsWeightedSumNode::DataIdx),
               true,
               NI.getInElemTy(FusedRowwiseQuantizedSparseLengthsWeightedSumNode::
                                  WeightsIdx),
               NI.getOutElemTy(
                   FusedRowwiseQuantizedSparseLengthsWeightedSumNode::
                       ResultIdx)) &&
           indexIs32or64(
               NI, FusedRowwiseQuantizedSparseLengthsWeightedSumNode::IndicesIdx) &&
           NI.getInElemTy(FusedRowwiseQuantizedSparseLengthsWeightedSumNode::
                              LengthsIdx) == ElemKind::Int32ITy;

  case Kinded::Kind::FusedRowwiseQuantizedSparseLengthsSumNodeKind:
    return fusedLookupTypesOk(
               NI.getInElemTy(
                   FusedRowwiseQuantizedSparseLengthsSumNode::DataIdx),
               false, ElemKind::FloatTy,
               NI.getOutElemTy(
                   FusedRowwiseQuantizedSparseLengthsSumNode::ResultIdx)) &&
           indexIs32or64(NI,
                         FusedRowwiseQuantizedSparseLengthsSumNode::IndicesIdx) &&
           NI.getInElemTy(FusedRowwiseQuantizedSparseLengthsSumNode::LengthsIdx) ==
               ElemKind::Int32ITy;

  case Kinded::Kind::RowwiseQuantizedSparseLengthsWeightedSumNodeKind:
    return NI.getInElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::DataIdx) ==
               ElemKind::UInt8QTy &&
           NI.getInElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::ScalesIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::OffsetsIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::WeightsIdx) ==
               ElemKind::FloatTy &&
           indexIs32or64(
               NI, RowwiseQuantizedSparseLengthsWeightedSumNode::IndicesIdx) &&
           NI.getInElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::LengthsIdx) ==
               ElemKind::Int32ITy &&
           NI.getOutElemTy(
               RowwiseQuantizedSparseLengthsWeightedSumNode::ResultIdx) ==
               ElemKind::FloatTy;

  case Kinded::Kind::EmbeddingBagByteRowwiseOffsetsNodeKind:
    return NI.getInElemTy(EmbeddingBagByteRowwiseOffsetsNode::DataIdx) ==
               ElemKind::UInt8FusedQTy &&
           NI.getInElemTy(EmbeddingBagByteRowwiseOffsetsNode::WeightsIdx) ==
               ElemKind::FloatTy &&
           NI.getInElemTy(EmbeddingBagByteRowwiseOffsetsNode::IndicesIdx) ==
               ElemKind::Int32ITy &&
           NI.getInElemTy(EmbeddingBagByteRowwiseOffsetsNode::OffsetsIdx) ==
               ElemKind::Int32ITy &&
           NI.getOutElemTy(EmbeddingBagByteRowwiseOffsetsNode::ResultIdx) ==
               ElemKind::FloatTy;

  // ---- int8 glue of a quantized image network --------------------------------
  case Kinded::Kind::AddNodeKind:       // ==> ElementAdd
  case Kinded::Kind::ReluNodeKind:      // stays un-lowered, ==> Relu
  case Kinded::Kind::ClipNodeKind:      // stays un-lowered, ==> Clip
  case Kinded::Kind::LeakyReluNodeKind: // stays un-lowered, ==> LeakyRelu
  case Kinded::Kind::AvgPoolNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy});

  // what a FullyConnected that some other pass lowered leaves behind its
  // MatMul (lib/Optimizer/Lower/Lower.cpp): int8 batch, int8 or int32 slice
  case Kinded::Kind::BatchedAddNodeKind:
    return NI.getInElemTy(BatchedAddNode::BatchIdx) == ElemKind::Int8QTy &&
           NI.getOutElemTy(BatchedAddNode::ResultIdx) == ElemKind::Int8QTy &&
           (NI.getInElemTy(BatchedAddNode::SliceIdx) == ElemKind::Int8QTy ||
            NI.getInElemTy(BatchedAddNode::SliceIdx) == ElemKind::Int32QTy);

#ifdef GLOW_WITH_CPU
  // Max(x, Splat(v)) as the CPU backend's node (the class exists when that
  // backend is built; transformPostLowering below makes it)
  case Kinded::Kind::CPUMaxSplatNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy});
#endif

  case Kinded::Kind::MaxPoolNodeKind:
    // the Argmax result is not produced: accepted only when it is unused,
    // which IRGen turns into the plain MaxPool instruction
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy}, {},
                                                  {MaxPoolNode::ArgmaxIdx});

  case Kinded::Kind::SoftMaxNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::FloatTy},
                                                  {SoftMaxNode::SelectedIdx});

  case Kinded::Kind::SigmoidNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::FloatTy});

  // ---- data movement of a ranking model --------------------------------------
  case Kinded::Kind::ConvertToNodeKind:
    return NI.getInElemTy(ConvertToNode::InputIdx) == ElemKind::Float16Ty &&
           NI.getOutElemTy(ConvertToNode::ResultIdx) == ElemKind::FloatTy;

  case Kinded::Kind::InsertTensorNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy});

  // any shuffle of up to six dimensions, any plain element kind
  // (libjit_transpose_i8 / _f / _u / _b, libjit.cpp:3162-3184)
  case Kinded::Kind::TransposeNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind(
        {ElemKind::Int8QTy, ElemKind::Int16QTy, ElemKind::Int32QTy, ElemKind::FloatTy,
         ElemKind::Float16Ty, ElemKind::Int32ITy, ElemKind::Int64ITy, ElemKind::BoolTy});

  case Kinded::Kind::GatherNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind({ElemKind::Int8QTy},
                                                  {GatherNode::IndicesIdx}) &&
           indexIs32or64(NI, GatherNode::IndicesIdx);

  // Reshape / Save / Flatten ==> TensorView or Copy of bytes: any kind the
  // path carries.
  case Kinded::Kind::SaveNodeKind:
  case Kinded::Kind::ReshapeNodeKind:
    return NI.allInputsAndOutputsHaveSameElemKind(
        {ElemKind::FloatTy, ElemKind::Float16Ty, ElemKind::Int8QTy,
         ElemKind::Int32QTy, ElemKind::Int32ITy, ElemKind::Int64ITy});

  default:
    return false;
  }
}

Expected<bool> MI355XBackend::transformPostLowering(
    Function *F, CompilationContext &cctx,
    const glow::runtime::DeviceInfo *devInfo) const {
  (void)cctx;
  (void)devInfo;
  bool changed = false;
#ifdef GLOW_WITH_CPU
  // Max(x, Splat(v)) on int8 of one type (a Relu that keeps its input's
  // parameters) becomes the CPU backend's CPUMaxSplatNode, as in
  // lib/Backends/CPU/Transforms.cpp: one elementwise pass instead of a Splat
  // tensor and a two-operand Max, for which this backend has no kernel.
  for (auto &node : F->getNodes()) {
    auto *MN = llvm::dyn_cast<MaxNode>(&node);
    if (!MN || MN->getResult().getElementType() != ElemKind::Int8QTy) {
      continue;
    }
    SplatNode *splat = llvm::dyn_cast<SplatNode>(MN->getLHS().getNode());
    NodeValue input = MN->getRHS();
    if (!splat) {
      splat = llvm::dyn_cast<SplatNode>(MN->getRHS().getNode());
      input = MN->getLHS();
    }
    if (!splat || input.getType() != MN->getResult().getType()) {
      continue;
    }
    auto *MS = F->addNode(new CPUMaxSplatNode(MN->getName(), input, splat->getValue()));
    MN->getResult().replaceAllUsesOfWith(MS->getResult());
    changed = true;
  }
#else
  (void)F;
#endif
  return changed;
}

bool MI355XBackend::shouldLower(const Node *N) const {
  switch (N->getKind()) {
  case Kinded::Kind::ReluNodeKind:
  case Kinded::Kind::ClipNodeKind:
  case Kinded::Kind::LeakyReluNodeKind:
  case Kinded::Kind::FullyConnectedNodeKind:
  case Kinded::Kind::ConvolutionNodeKind:
  // the plain Sum has a kernel path of its own (weights == NULL); lowering it
  // would materialise a Splat(1.0) weights tensor per lookup
  // (lib/Optimizer/Lower/Lower.cpp:1590-1606)
  case Kinded::Kind::FusedRowwiseQuantizedSparseLengthsSumNodeKind:
  // one launch for the whole batch instead of one MatMul per sample
  case Kinded::Kind::BatchMatMulNodeKind:
    return false;
  default:
    return true;
  }
}

bool MI355XBackend::supportsFusedActivation(Node *parent,
                                            Node *activation) const {
  if (!llvm::isa<ConvolutionNode>(parent) &&
      !llvm::isa<ChannelwiseQuantizedConvolutionNode>(parent)) {
    return false;
  }
  switch (activation->getKind()) {
  case Kinded::Kind::ReluNodeKind:
  case Kinded::Kind::ClipNodeKind:
  case Kinded::Kind::LeakyReluNodeKind:
    return true;
  default:
    // quantized Sigmoid / Tanh arrive as lookup tables, never fused
    return false;
  }
}

bool MI355XBackend::canDoIndexTypeDemotion(
    ElemKind fromTy, ElemKind toTy, PrecisionConfiguration &precConfig) const {
  precConfig.precisionModeKindSet.insert(
      Kinded::Kind::EmbeddingBagByteRowwiseOffsetsNodeKind);
  precConfig.precisionModeKindSet.insert(
      Kinded::Kind::FusedRowwiseQuantizedSparseLengthsSumNodeKind);
  precConfig.precisionModeKindSet.insert(
      Kinded::Kind::FusedRowwiseQuantizedSparseLengthsWeightedSumNodeKind);
  precConfig.precisionModeKindSet.insert(
      Kinded::Kind::RowwiseQuantizedSparseLengthsWeightedSumNodeKind);
  return fromTy == ElemKind::Int64ITy && toTy == ElemKind::Int32ITy;
}

runtime::DeviceManager *
MI355XBackend::createDeviceManager(const runtime::DeviceConfig &deviceConfig) {
  return runtime::createMI355XDeviceManager(deviceConfig);
}

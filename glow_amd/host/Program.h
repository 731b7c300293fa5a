// The lowered program the backend compiles: a module of constants and
// placeholders, and functions that are straight-line lists of instructions
// over statically planned buffers. It restates, at the level the hot path
// needs, what glow::Module / glow::IRFunction / glow::runtime::RuntimeBundle
// hand to a backend (reference include/glow/IR/IR.h, tools/ClassGen/InstrGen.cpp
// for operand order, lib/Backends/BackendUtils.cpp:702-730 for the three-region
// memory plan). Inside a Glow build the same information is read off the real
// IRFunction; see the MI355X backend notes shipped with this library.
#ifndef GLOW_MI355X_HOST_PROGRAM_H
#define GLOW_MI355X_HOST_PROGRAM_H

#include "Error.h"
#include "Type.h"

#include <map>
#include <memory>
#include <string>
#include <vector>

namespace glow_mi355x {

constexpr size_t kTensorAlignment = 64; // glow::TensorAlignment (Support/Memory.h:29)

// RuntimeSymbolInfo::symbolCategory (BackendUtils.h:41-62)
enum class SymbolCategory : int32_t { Constant = 0, Placeholder, Activation };

struct Value {
  int id = -1;
  std::string name;
  Type type;
  SymbolCategory category = SymbolCategory::Activation;
  size_t offset = 0; // byte offset inside the region of its category
  int function = -1; // owning function for activations
  int root = -1;     // the value whose memory this one is a view of (itself if none)
};

// Instruction kinds: the names are Glow's IR instruction names without "Inst".
enum class Kind : int32_t {
  Quantize = 0,                 // (Dest, Src)
  Dequantize,                   // (Dest, Src)
  RescaleQuantized,             // (Dest, Src)
  FullyConnected,               // (Dest, Src, Weights[K,N], Bias)
  RowwiseQuantizedFullyConnected, // (Dest, Src, Weights[N,K], Bias, Scales, Offsets)
  MatMul,                       // (Dest, LHS, RHS)
  Convolution,                  // (Dest, Src, Filter, Bias) + conv attributes
  ChannelwiseQuantizedConvolution, // (Dest, Src, Filter, Bias, FilterScales, FilterOffsets, BiasScales, BiasOffsets) + conv attributes
  FusedRowwiseQuantizedSparseLengthsWeightedSum, // (Dest, Data, Weights, Indices, Lengths); iattrs {useFP16Accumulation}
  FusedRowwiseQuantizedSparseLengthsSum,         // (Dest, Data, Indices, Lengths); iattrs {useFP16Accumulation}
  ElementAdd,                   // (Dest, LHS, RHS)
  Relu,                         // (Dest, Src)
  MaxPool,                      // (Dest, Src); iattrs {kernelH, kernelW, strideH, strideW, padT, padL, padB, padR}
  AvgPool,                      // (Dest, Src); MaxPool's iattrs + {countIncludePads}
  SoftMax,                      // (Dest, Src), float [rows x cols]
  ConvertTo,                    // (Result float, Input float16)
  InsertTensor,                 // (Dest [R,W], Src [R,w]); iattrs {offset in the inner dimension}
  Transpose,                    // (Dest, Src) int8; iattrs = shuffle, {1,0} or {0,2,1}
  Gather,                       // (Dest, Data, Indices); iattrs {batchDims (0 or 1)}
  BatchMatMul,                  // (Dest [B,M,N], LHS [B,M,K], RHS [B,K,N]) int8
  Sigmoid,                      // (Dest, Src) float
  RowwiseQuantizedSparseLengthsWeightedSum, // (Dest, Data u8 [rows,cols], Scales, Offsets, Weights, Indices, Lengths)
  EmbeddingBagByteRowwiseOffsets, // (Dest, Data, Weights, Indices, Offsets); iattrs {hasEndOffset}
  Copy,                         // (Dest, Src): same bytes (what Save and Reshape lower to)
  Clip,                         // (Dest, Src) int8; fattrs {min, max}
  LeakyRelu,                    // (Dest, Src) int8; fattrs {alpha}
  CPUMaxSplat,                  // (Dest, Src) int8 of one type; fattrs {splatValue}: max(x, splat)
  BatchedAdd,                   // (Dest, Batch, Slice) int8 batch; slice int8 or int32
  NumKinds
};
const char *kindName(Kind k);

// Nodes.h:276-283
enum FusedActivation : int32_t { NONE = 0, RELU, CLIP, TANH, SIGMOID, LEAKY_RELU };

// Integer attributes of the two convolution kinds, in this order.
struct ConvAttrs {
  int64_t kernelH, kernelW, strideH, strideW;
  int64_t padT, padL, padB, padR; // Glow's TLBR
  int64_t group, dilationH, dilationW;
  int64_t fusedActivation;        // FusedActivation
  static constexpr int kCount = 12;
};

struct Instruction {
  Kind kind;
  std::string name;
  std::vector<int> operands;   // value ids, in the reference's operand order
  std::vector<int64_t> iattrs;
  std::vector<float> fattrs;   // fused activation arguments (float, as in the node)
};

class Module;

class Function {
public:
  Function(Module *m, int index, std::string name)
      : module_(m), index_(index), name_(std::move(name)) {}
  const std::string &name() const { return name_; }
  Module *module() const { return module_; }
  int index() const { return index_; }

  // AllocActivationInst
  int createActivation(const std::string &name, const Type &t);
  int addInstruction(Kind kind, const std::string &name, std::vector<int> operands,
                     std::vector<int64_t> iattrs = {}, std::vector<float> fattrs = {});

  // Builder shorthands in the reference's operand order.
  int createQuantize(const std::string &n, int dest, int src) {
    return addInstruction(Kind::Quantize, n, {dest, src});
  }
  int createDequantize(const std::string &n, int dest, int src) {
    return addInstruction(Kind::Dequantize, n, {dest, src});
  }
  int createRescaleQuantized(const std::string &n, int dest, int src) {
    return addInstruction(Kind::RescaleQuantized, n, {dest, src});
  }
  int createFullyConnected(const std::string &n, int dest, int src, int weights, int bias) {
    return addInstruction(Kind::FullyConnected, n, {dest, src, weights, bias});
  }
  int createRowwiseQuantizedFullyConnected(const std::string &n, int dest, int src,
                                           int weights, int bias, int scales,
                                           int offsets) {
    return addInstruction(Kind::RowwiseQuantizedFullyConnected, n,
                          {dest, src, weights, bias, scales, offsets});
  }
  int createMatMul(const std::string &n, int dest, int lhs, int rhs) {
    return addInstruction(Kind::MatMul, n, {dest, lhs, rhs});
  }
  int createConvolution(const std::string &n, int dest, int src, int filter, int bias,
                        const ConvAttrs &a, std::vector<float> actArgs = {});
  int createChannelwiseQuantizedConvolution(const std::string &n, int dest, int src,
                                            int filter, int bias, int filterScales,
                                            int filterOffsets, int biasScales,
                                            int biasOffsets, const ConvAttrs &a,
                                            std::vector<float> actArgs = {});
  int createFusedRowwiseQuantizedSparseLengthsWeightedSum(const std::string &n, int dest,
                                                          int data, int weights,
                                                          int indices, int lengths,
                                                          bool useFP16Accumulation = false) {
    return addInstruction(Kind::FusedRowwiseQuantizedSparseLengthsWeightedSum, n,
                          {dest, data, weights, indices, lengths},
                          {useFP16Accumulation ? 1 : 0});
  }
  int createFusedRowwiseQuantizedSparseLengthsSum(const std::string &n, int dest, int data,
                                                  int indices, int lengths,
                                                  bool useFP16Accumulation = false) {
    return addInstruction(Kind::FusedRowwiseQuantizedSparseLengthsSum, n,
                          {dest, data, indices, lengths},
                          {useFP16Accumulation ? 1 : 0});
  }

  const std::vector<Instruction> &instructions() const { return insts_; }
  size_t activationsSize() const { return actSize_; }

private:
  Module *module_;
  int index_;
  std::string name_;
  std::vector<Instruction> insts_;
  size_t actSize_ = 0;
};

class Module {
public:
  explicit Module(std::string name = "module") : name_(std::move(name)) {}
  const std::string &name() const { return name_; }

  // Module::createConstant: the payload is copied.
  int createConstant(const std::string &name, const Type &t, const void *payload);
  // Module::createPlaceholder
  int createPlaceholder(const std::string &name, const Type &t);
  Function *createFunction(const std::string &name);
  // TensorViewInst: another type over the bytes of `src` from `byteOffset` on (a
  // reshape, or a slice of the outermost dimension); the view must lie inside
  // its source. Returns -1 when it does not, or when a view that does not
  // start at its source's first byte is asked of an activation (activations are
  // placed by the backend; placeholders and constants have fixed offsets).
  int createView(const std::string &name, int src, const Type &t, size_t byteOffset = 0);

  const Value &value(int id) const { return values_.at((size_t)id); }
  bool validId(int id) const { return id >= 0 && (size_t)id < values_.size(); }
  int numValues() const { return (int)values_.size(); }
  int getValueByName(const std::string &name) const; // -1 if absent
  Function *getFunction(const std::string &name) const;
  const std::vector<std::unique_ptr<Function>> &functions() const { return funcs_; }

  size_t constantsSize() const { return constSize_; }
  size_t mutableSize() const { return mutSize_; }
  // host image of the constants region (what collectConstants builds,
  // BackendUtils.cpp:62-106)
  const std::vector<uint8_t> &constantsImage() const { return constImage_; }

private:
  friend class Function;
  int addValue(Value v);
  std::string name_;
  std::vector<Value> values_;
  std::vector<std::unique_ptr<Function>> funcs_;
  std::vector<uint8_t> constImage_;
  size_t constSize_ = 0, mutSize_ = 0;
};

inline size_t alignUp(size_t v, size_t a) { return (v + a - 1) / a * a; }

} // namespace glow_mi355x
#endif

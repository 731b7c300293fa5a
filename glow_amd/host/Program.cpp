#include "Program.h"

#include <cstdarg>
#include <cstdio>

namespace glow_mi355x {

const char *errorCodeName(ErrorCode c) {
  switch (c) {
  case ErrorCode::SUCCESS: return "SUCCESS";
  case ErrorCode::UNKNOWN: return "UNKNOWN";
  case ErrorCode::RUNTIME_ERROR: return "RUNTIME_ERROR";
  case ErrorCode::RUNTIME_OUT_OF_DEVICE_MEMORY: return "RUNTIME_OUT_OF_DEVICE_MEMORY";
  case ErrorCode::RUNTIME_NET_NOT_FOUND: return "RUNTIME_NET_NOT_FOUND";
  case ErrorCode::RUNTIME_REQUEST_REFUSED: return "RUNTIME_REQUEST_REFUSED";
  case ErrorCode::RUNTIME_DEVICE_NOT_FOUND: return "RUNTIME_DEVICE_NOT_FOUND";
  case ErrorCode::RUNTIME_DEVICE_NONRECOVERABLE: return "RUNTIME_DEVICE_NONRECOVERABLE";
  case ErrorCode::RUNTIME_NET_BUSY: return "RUNTIME_NET_BUSY";
  case ErrorCode::DEVICE_FEATURE_NOT_SUPPORTED: return "DEVICE_FEATURE_NOT_SUPPORTED";
  case ErrorCode::COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE:
    return "COMPILE_UNSUPPORTED_NODE_AFTER_OPTIMIZE";
  case ErrorCode::COMPILE_CONTEXT_MALFORMED: return "COMPILE_CONTEXT_MALFORMED";
  }
  return "UNKNOWN";
}

std::string Error::str() const {
  if (code_ == ErrorCode::SUCCESS) return "success";
  return std::string(errorCodeName(code_)) + ": " + msg_;
}

std::string strFormat(const char *fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  return buf;
}

const char *elemKindName(ElemKind k) {
  switch (k) {
  case ElemKind::FloatTy: return "float";
  case ElemKind::Float16Ty: return "float16";
  case ElemKind::Int8QTy: return "i8";
  case ElemKind::Int32QTy: return "i32";
  case ElemKind::Int32ITy: return "index32";
  case ElemKind::Int64ITy: return "index64";
  case ElemKind::UInt8FusedQTy: return "ui8fused";
  case ElemKind::UInt8FusedFP16QTy: return "ui8fusedfp16";
  case ElemKind::UInt4FusedFP16QTy: return "ui4fusedfp16";
  case ElemKind::UInt4FusedQTy: return "ui4fused";
  case ElemKind::BoolTy: return "bool";
  case ElemKind::Int16QTy: return "i16";
  }
  return "?";
}

size_t elemSize(ElemKind k) {
  switch (k) {
  case ElemKind::FloatTy: case ElemKind::Int32QTy: case ElemKind::Int32ITy: return 4;
  case ElemKind::Float16Ty: case ElemKind::Int16QTy: return 2;
  case ElemKind::Int64ITy: return 8;
  default: return 1;
  }
}

std::string Type::str() const {
  std::string s = elemKindName(kind);
  if (isQuantized(kind)) s += strFormat("[S:%g O:%d]", (double)scale, offset);
  s += "<";
  for (size_t i = 0; i < dims.size(); i++)
    s += (i ? " x " : "") + std::to_string(dims[i]);
  return s + ">";
}

const char *kindName(Kind k) {
  switch (k) {
  case Kind::Quantize: return "Quantize";
  case Kind::Dequantize: return "Dequantize";
  case Kind::RescaleQuantized: return "RescaleQuantized";
  case Kind::FullyConnected: return "FullyConnected";
  case Kind::RowwiseQuantizedFullyConnected: return "RowwiseQuantizedFullyConnected";
  case Kind::MatMul: return "MatMul";
  case Kind::Convolution: return "Convolution";
  case Kind::ChannelwiseQuantizedConvolution: return "ChannelwiseQuantizedConvolution";
  case Kind::FusedRowwiseQuantizedSparseLengthsWeightedSum:
    return "FusedRowwiseQuantizedSparseLengthsWeightedSum";
  case Kind::FusedRowwiseQuantizedSparseLengthsSum:
    return "FusedRowwiseQuantizedSparseLengthsSum";
  case Kind::ElementAdd: return "ElementAdd";
  case Kind::Relu: return "Relu";
  case Kind::MaxPool: return "MaxPool";
  case Kind::AvgPool: return "AvgPool";
  case Kind::SoftMax: return "SoftMax";
  case Kind::ConvertTo: return "ConvertTo";
  case Kind::InsertTensor: return "InsertTensor";
  case Kind::Transpose: return "Transpose";
  case Kind::Gather: return "Gather";
  case Kind::BatchMatMul: return "BatchMatMul";
  case Kind::Sigmoid: return "Sigmoid";
  case Kind::RowwiseQuantizedSparseLengthsWeightedSum: return "RowwiseQuantizedSparseLengthsWeightedSum";
  case Kind::EmbeddingBagByteRowwiseOffsets: return "EmbeddingBagByteRowwiseOffsets";
  case Kind::Copy: return "Copy";
  case Kind::Clip: return "Clip";
  case Kind::LeakyRelu: return "LeakyRelu";
  case Kind::CPUMaxSplat: return "CPUMaxSplat";
  case Kind::BatchedAdd: return "BatchedAdd";
  default: return "?";
  }
}

int Module::createView(const std::string &name, int src, const Type &t, size_t byteOffset) {
  if (!validId(src)) return -1;
  const Value &s = values_[(size_t)src];
  if (byteOffset > s.type.sizeInBytes() || t.sizeInBytes() > s.type.sizeInBytes() - byteOffset)
    return -1;
  if (byteOffset != 0 && s.category == SymbolCategory::Activation) return -1;
  Value v;
  v.name = name;
  v.type = t;
  v.category = s.category;
  v.offset = s.offset + byteOffset;
  v.function = s.function;
  v.root = s.root;
  return addValue(std::move(v));
}

int Module::addValue(Value v) {
  v.id = (int)values_.size();
  if (v.root < 0) v.root = v.id;
  values_.push_back(std::move(v));
  return values_.back().id;
}

int Module::createConstant(const std::string &name, const Type &t, const void *payload) {
  Value v;
  v.name = name;
  v.type = t;
  v.category = SymbolCategory::Constant;
  v.offset = constSize_;
  const size_t n = t.sizeInBytes();
  constSize_ = alignUp(constSize_ + n, kTensorAlignment);
  constImage_.resize(constSize_, 0);
  if (payload && n) std::memcpy(constImage_.data() + v.offset, payload, n);
  return addValue(std::move(v));
}

int Module::createPlaceholder(const std::string &name, const Type &t) {
  Value v;
  v.name = name;
  v.type = t;
  v.category = SymbolCategory::Placeholder;
  v.offset = mutSize_;
  mutSize_ = alignUp(mutSize_ + t.sizeInBytes(), kTensorAlignment);
  return addValue(std::move(v));
}

Function *Module::createFunction(const std::string &name) {
  funcs_.emplace_back(new Function(this, (int)funcs_.size(), name));
  return funcs_.back().get();
}

int Module::getValueByName(const std::string &name) const {
  for (const auto &v : values_)
    if (v.name == name) return v.id;
  return -1;
}

Function *Module::getFunction(const std::string &name) const {
  for (const auto &f : funcs_)
    if (f->name() == name) return f.get();
  return nullptr;
}

int Function::createActivation(const std::string &name, const Type &t) {
  Value v;
  v.name = name;
  v.type = t;
  v.category = SymbolCategory::Activation;
  v.function = index_;
  v.offset = actSize_;
  actSize_ = alignUp(actSize_ + t.sizeInBytes(), kTensorAlignment);
  return module_->addValue(std::move(v));
}

int Function::addInstruction(Kind kind, const std::string &name, std::vector<int> operands,
                             std::vector<int64_t> iattrs, std::vector<float> fattrs) {
  Instruction I;
  I.kind = kind;
  I.name = name;
  I.operands = std::move(operands);
  I.iattrs = std::move(iattrs);
  I.fattrs = std::move(fattrs);
  insts_.push_back(std::move(I));
  return (int)insts_.size() - 1;
}

static std::vector<int64_t> convIattrs(const ConvAttrs &a) {
  return {a.kernelH, a.kernelW, a.strideH, a.strideW, a.padT, a.padL, a.padB,
          a.padR, a.group, a.dilationH, a.dilationW, a.fusedActivation};
}

int Function::createConvolution(const std::string &n, int dest, int src, int filter,
                                int bias, const ConvAttrs &a, std::vector<float> actArgs) {
  return addInstruction(Kind::Convolution, n, {dest, src, filter, bias}, convIattrs(a),
                        std::move(actArgs));
}

int Function::createChannelwiseQuantizedConvolution(
    const std::string &n, int dest, int src, int filter, int bias, int filterScales,
    int filterOffsets, int biasScales, int biasOffsets, const ConvAttrs &a,
    std::vector<float> actArgs) {
  return addInstruction(Kind::ChannelwiseQuantizedConvolution, n,
                        {dest, src, filter, bias, filterScales, filterOffsets,
                         biasScales, biasOffsets},
                        convIattrs(a), std::move(actArgs));
}

} // namespace glow_mi355x

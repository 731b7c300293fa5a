// Tensor types and host tensors as the hot path sees them: the subset of
// glow::ElemKind / glow::Type / glow::Tensor (reference include/glow/Base/Type.h:401-473,
// include/glow/Base/Tensor.h) that lowered quantized instructions carry.
#ifndef GLOW_MI355X_HOST_TYPE_H
#define GLOW_MI355X_HOST_TYPE_H

#include <cstddef>
#include <cstdint>
#include <cstring>
#include <string>
#include <vector>

namespace glow_mi355x {

// Numbering is this library's own; names are Glow's.
enum class ElemKind : int32_t {
  FloatTy = 0,
  Float16Ty,
  Int8QTy,
  Int32QTy,
  Int32ITy,
  Int64ITy,
  UInt8FusedQTy,      // u8 data, fp32 scale+offset at the row end
  UInt8FusedFP16QTy,  // u8 data, fp16 scale+offset
  UInt4FusedFP16QTy,  // u4 data, fp16 scale+offset
  UInt4FusedQTy,      // u4 data, fp32 scale+offset
  BoolTy,
  Int16QTy,
};

const char *elemKindName(ElemKind k);
size_t elemSize(ElemKind k);
inline bool isQuantized(ElemKind k) {
  return k == ElemKind::Int8QTy || k == ElemKind::Int32QTy || k == ElemKind::Int16QTy;
}
inline bool isFused(ElemKind k) {
  return k == ElemKind::UInt8FusedQTy || k == ElemKind::UInt8FusedFP16QTy ||
         k == ElemKind::UInt4FusedFP16QTy || k == ElemKind::UInt4FusedQTy;
}

struct Type {
  ElemKind kind = ElemKind::FloatTy;
  std::vector<int64_t> dims;
  float scale = 1.0f;   // quantized kinds only
  int32_t offset = 0;

  Type() = default;
  Type(ElemKind k, std::vector<int64_t> d, float s = 1.0f, int32_t o = 0)
      : kind(k), dims(std::move(d)), scale(s), offset(o) {}
  int64_t size() const {
    int64_t n = 1;
    for (auto d : dims) n *= d;
    return n;
  }
  size_t sizeInBytes() const { return (size_t)size() * elemSize(kind); }
  std::string str() const;
};

// Host tensor: a type and its bytes, owned or (unowned) borrowed from the caller.
class Tensor {
public:
  Tensor() = default;
  explicit Tensor(Type t) : type_(std::move(t)), bytes_(type_.sizeInBytes()) {
    ptr_ = bytes_.data();
    size_ = bytes_.size();
  }
  Tensor(Type t, const void *data) : Tensor(std::move(t)) {
    if (size_) std::memcpy(ptr_, data, size_);
  }
  // Tensor(void *data, TypeRef ty): a view of caller memory of `bytes` bytes
  static Tensor unowned(Type t, void *data, size_t bytes) {
    Tensor r;
    r.type_ = std::move(t);
    r.ptr_ = static_cast<uint8_t *>(data);
    r.size_ = bytes;
    return r;
  }
  Tensor(Tensor &&o) noexcept { *this = std::move(o); }
  Tensor &operator=(Tensor &&o) noexcept {
    const bool owned = !o.bytes_.empty() && o.ptr_ == o.bytes_.data();
    type_ = std::move(o.type_);
    bytes_ = std::move(o.bytes_);
    ptr_ = owned ? bytes_.data() : o.ptr_;
    size_ = o.size_;
    o.ptr_ = nullptr;
    o.size_ = 0;
    return *this;
  }
  Tensor(const Tensor &) = delete;
  Tensor &operator=(const Tensor &) = delete;
  const Type &type() const { return type_; }
  size_t sizeInBytes() const { return size_; }
  void *data() { return ptr_; }
  const void *data() const { return ptr_; }

private:
  Type type_;
  std::vector<uint8_t> bytes_;
  uint8_t *ptr_ = nullptr;
  size_t size_ = 0;
};

} // namespace glow_mi355x
#endif

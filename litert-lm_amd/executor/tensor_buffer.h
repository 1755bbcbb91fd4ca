// Host tensor handle that stands in for litert::TensorBuffer at the executor
// boundary (LiteRT's headers are not available outside the reference's Bazel
// workspace). It keeps what the executor interface relies on
// (runtime/util/convert_tensor_buffer.h:62-229): typed dims, host-visible
// memory, and Duplicate() handing out another reference to the same storage.
#ifndef LITERT_LM_AMD_EXECUTOR_TENSOR_BUFFER_H_
#define LITERT_LM_AMD_EXECUTOR_TENSOR_BUFFER_H_

#include <cstdint>
#include <cstring>
#include <memory>
#include <vector>

#include "status.h"

namespace litert::lm {

enum class ElementType { kNone, kInt32, kFloat32, kFloat16, kBool };

inline size_t ElementSize(ElementType t) {
  switch (t) {
    case ElementType::kInt32:
    case ElementType::kFloat32: return 4;
    case ElementType::kFloat16: return 2;
    case ElementType::kBool: return 1;
    default: return 0;
  }
}

class TensorBuffer {
 public:
  TensorBuffer() = default;

  static TensorBuffer Create(ElementType type, std::vector<int> dims) {
    TensorBuffer t;
    t.type_ = type;
    t.dims_ = std::move(dims);
    t.storage_ = std::make_shared<std::vector<uint8_t>>(t.PackedSize(), 0);
    return t;
  }
  template <class T>
  static TensorBuffer CopyFrom(ElementType type, std::vector<int> dims, const T* data) {
    TensorBuffer t = Create(type, std::move(dims));
    std::memcpy(t.data(), data, t.PackedSize());
    return t;
  }

  bool HasValue() const { return storage_ != nullptr; }
  ElementType type() const { return type_; }
  const std::vector<int>& dims() const { return dims_; }
  size_t NumElements() const {
    size_t n = storage_ ? 1 : 0;
    for (int d : dims_) n *= static_cast<size_t>(d);
    return n;
  }
  size_t PackedSize() const {
    size_t n = 1;
    for (int d : dims_) n *= static_cast<size_t>(d);
    return n * ElementSize(type_);
  }
  void* data() { return storage_ ? storage_->data() : nullptr; }
  const void* data() const { return storage_ ? storage_->data() : nullptr; }
  template <class T>
  T* as() { return static_cast<T*>(data()); }
  template <class T>
  const T* as() const { return static_cast<const T*>(data()); }

  // Another handle to the same memory (reference-counted).
  TensorBuffer Duplicate() const { return *this; }

 private:
  ElementType type_ = ElementType::kNone;
  std::vector<int> dims_;
  std::shared_ptr<std::vector<uint8_t>> storage_;
};

}  // namespace litert::lm
#endif  // LITERT_LM_AMD_EXECUTOR_TENSOR_BUFFER_H_

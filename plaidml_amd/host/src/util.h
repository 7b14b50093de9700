// Element types, tensor shapes, host buffers and settings of the host library.
//
// Restates pmlc/util/{enums.td:35-57, shape.h:16-39, shape.cc:11-103, buffer.h:15-88}
// and plaidml/core/settings.cc:19-87 of the reference without MLIR.
#pragma once

#include <cstdint>
#include <cstring>
#include <map>
#include <memory>
#include <new>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

namespace pmlc::util {

// Numeric values follow plaidml_datatype; the order is also the promotion score
// (pmlc/dialect/tile/ir/util.cc:44-100).  bf16 is appended.
enum class DataType : int {
  invalid = 0,
  six = 1,
  uix = 2,
  fx = 3,
  i1 = 4,
  si8 = 5,
  ui8 = 6,
  si16 = 7,
  ui16 = 8,
  si32 = 9,
  ui32 = 10,
  si64 = 11,
  ui64 = 12,
  f16 = 13,
  f32 = 14,
  f64 = 15,
  bf16 = 16,
};

inline const char* mnemonic(DataType dt) {
  static const char* names[] = {"invalid", "six",  "uix",  "fx",   "i1",  "si8", "ui8", "si16", "ui16",
                                "si32",    "ui32", "si64", "ui64", "f16", "f32", "f64", "bf16"};
  int i = static_cast<int>(dt);
  return (i >= 0 && i <= 16) ? names[i] : "invalid";
}

inline bool isFloat(DataType dt) {
  return dt == DataType::f16 || dt == DataType::f32 || dt == DataType::f64 || dt == DataType::bf16 || dt == DataType::fx;
}
inline bool isSigned(DataType dt) {
  return dt == DataType::si8 || dt == DataType::si16 || dt == DataType::si32 || dt == DataType::si64 || dt == DataType::six;
}
inline bool isUnsigned(DataType dt) {
  return dt == DataType::ui8 || dt == DataType::ui16 || dt == DataType::ui32 || dt == DataType::ui64 || dt == DataType::uix;
}
inline bool isInteger(DataType dt) { return isSigned(dt) || isUnsigned(dt) || dt == DataType::i1; }
inline bool isAmbiguous(DataType dt) { return dt == DataType::six || dt == DataType::uix || dt == DataType::fx; }

// Promotion score: enum order, with bf16 declared to sit between f16 and f32.
inline double typeScore(DataType dt) { return dt == DataType::bf16 ? 13.5 : static_cast<double>(static_cast<int>(dt)); }
inline DataType promoteTypes(DataType a, DataType b) { return typeScore(a) > typeScore(b) ? a : b; }

inline size_t byteSize(DataType dt) {
  switch (dt) {
    case DataType::i1:
    case DataType::si8:
    case DataType::ui8:
      return 1;
    case DataType::si16:
    case DataType::ui16:
    case DataType::f16:
    case DataType::bf16:
      return 2;
    case DataType::si32:
    case DataType::ui32:
    case DataType::f32:
      return 4;
    case DataType::si64:
    case DataType::ui64:
    case DataType::f64:
      return 8;
    default:
      return 0;
  }
}

struct TensorShape {
  DataType elementType = DataType::invalid;
  std::vector<int64_t> sizes;
  std::vector<int64_t> strides;  // empty = dense row-major

  TensorShape() = default;
  explicit TensorShape(DataType dt) : elementType(dt) {}
  TensorShape(DataType dt, std::vector<int64_t> s) : elementType(dt), sizes(std::move(s)) {}
  TensorShape(DataType dt, std::vector<int64_t> s, std::vector<int64_t> st)
      : elementType(dt), sizes(std::move(s)), strides(std::move(st)) {}

  size_t getRank() const { return sizes.size(); }
  int64_t elements() const {
    int64_t n = 1;
    for (int64_t s : sizes) n *= s;
    return n;
  }
  std::vector<int64_t> denseStrides() const {
    std::vector<int64_t> st(sizes.size());
    int64_t s = 1;
    for (int i = static_cast<int>(sizes.size()) - 1; i >= 0; --i) {
      st[i] = s;
      s *= sizes[i];
    }
    return st;
  }
  size_t getByteSize() const {
    if (strides.empty()) return static_cast<size_t>(elements()) * byteSize(elementType);
    int64_t total = 1;
    for (size_t i = 0; i < sizes.size(); ++i) {
      if (!sizes[i]) return 0;
      total += (sizes[i] - 1) * strides[i];
    }
    return static_cast<size_t>(total) * byteSize(elementType);
  }
  // "8x32xf32", rank 0 -> "f32", unknown dim -> "?", explicit strides appended as ", [s0xs1]"
  std::string str() const {
    std::stringstream ss;
    for (int64_t d : sizes) {
      if (d)
        ss << d;
      else
        ss << '?';
      ss << 'x';
    }
    ss << mnemonic(elementType);
    if (!strides.empty()) {
      ss << ", [";
      for (size_t i = 0; i < strides.size(); ++i) {
        if (i) ss << 'x';
        ss << strides[i];
      }
      ss << ']';
    }
    return ss.str();
  }
  bool operator==(const TensorShape& rhs) const {
    return elementType == rhs.elementType && sizes == rhs.sizes && strides == rhs.strides;
  }
  bool operator!=(const TensorShape& rhs) const { return !(*this == rhs); }
};

using TensorShapes = std::vector<TensorShape>;

// Host memory seen through the API.  A device backend treats every buffer as
// host memory that may change between runs.
class Buffer {
 public:
  virtual ~Buffer() = default;
  virtual char* data() = 0;
  virtual size_t size() const = 0;
  virtual std::shared_ptr<Buffer> clone() = 0;
  const TensorShape& shape() const { return shape_; }

 protected:
  explicit Buffer(TensorShape shape) : shape_(std::move(shape)) {}
  TensorShape shape_;
};
using BufferPtr = std::shared_ptr<Buffer>;

// owns zero-initialised storage
class SimpleBuffer : public Buffer, public std::enable_shared_from_this<SimpleBuffer> {
 public:
  explicit SimpleBuffer(const TensorShape& shape) : Buffer(shape), data_(shape.getByteSize()) {}
  SimpleBuffer(const TensorShape& shape, std::vector<char> data) : Buffer(shape), data_(std::move(data)) {}
  char* data() final { return data_.data(); }
  size_t size() const final { return data_.size(); }
  BufferPtr clone() final { return std::make_shared<SimpleBuffer>(shape_, data_); }

 private:
  std::vector<char> data_;
};

// owns zero-initialised storage obtained from (and returned to) a caller-given pair of functions: page-locked
// host memory when a GPU is present
class ForeignBuffer : public Buffer {
 public:
  typedef void* (*AllocFn)(size_t);
  typedef void (*FreeFn)(void*);
  // throws std::bad_alloc when `alloc` returns nullptr
  ForeignBuffer(const TensorShape& shape, AllocFn alloc, FreeFn release)
      : Buffer(shape), size_(shape.getByteSize()), alloc_(alloc), release_(release) {
    data_ = static_cast<char*>(alloc_(size_ ? size_ : 1));
    if (!data_) throw std::bad_alloc();
  }
  ~ForeignBuffer() override { release_(data_); }
  ForeignBuffer(const ForeignBuffer&) = delete;
  ForeignBuffer& operator=(const ForeignBuffer&) = delete;
  char* data() final { return data_; }
  size_t size() const final { return size_; }
  BufferPtr clone() final {
    try {
      auto copy = std::make_shared<ForeignBuffer>(shape_, alloc_, release_);
      std::memcpy(copy->data_, data_, size_);
      return copy;
    } catch (const std::bad_alloc&) {  // the allocator has no more to give (a cap on page-locked memory): ordinary memory
      auto copy = std::make_shared<SimpleBuffer>(shape_);
      std::memcpy(copy->data(), data_, size_);
      return copy;
    }
  }

 private:
  char* data_ = nullptr;
  size_t size_;
  AllocFn alloc_;
  FreeFn release_;
};

// aliases caller memory: no copy, no ownership
class AdoptedBuffer : public Buffer {
 public:
  AdoptedBuffer(const TensorShape& shape, char* data, size_t size) : Buffer(shape), data_(data), size_(size) {}
  char* data() final { return data_; }
  size_t size() const final { return size_; }
  BufferPtr clone() final { return std::make_shared<AdoptedBuffer>(shape_, data_, size_); }

 private:
  char* data_;
  size_t size_;
};

// Settings: an environment variable wins over the settings file.
class Settings {
 public:
  static Settings* Instance();
  std::string get(const std::string& key) const;
  void set(const std::string& key, const std::string& value);
  const std::map<std::string, std::string>& all() const { return settings_; }
  void load();
  void save();

 private:
  std::map<std::string, std::string> settings_;
};

std::string getEnvVar(const std::string& key, const std::string& def = "");
int verbosity();

}  // namespace pmlc::util

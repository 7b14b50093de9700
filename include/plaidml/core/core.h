// C++ view of the core C ABI: DType, TensorShape, Buffer, Program, Settings.
// Same class and method names as the reference header (plaidml/core/core.h:101-470)
// so that Tile programs written against it compile unchanged; every object is a
// shared handle released through the matching plaidml_*_free.
#pragma once

#include <cstring>
#include <memory>
#include <ostream>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "plaidml/core/ffi.h"

namespace plaidml {

// Thrown when a C ABI call reports an error.
class ffi_exception : public std::runtime_error {
 public:
  explicit ffi_exception(const std::string& what) : std::runtime_error(what) {}
};

namespace ffi {

inline std::string str(plaidml_string* ptr) {
  std::string ret = ptr ? plaidml_string_ptr(ptr) : "";
  if (ptr) plaidml_string_free(ptr);
  return ret;
}

inline void rethrow(plaidml_error* err) {
  if (err->code) throw ffi_exception(str(err->msg));
}

// call<T>(fn, args...) invokes fn(&err, args...) and throws on failure
template <typename T, typename F, typename... Args>
T call(F fn, Args... args) {
  plaidml_error err{0, nullptr};
  T ret = fn(&err, args...);
  rethrow(&err);
  return ret;
}

template <typename F, typename... Args>
void call_void(F fn, Args... args) {
  plaidml_error err{0, nullptr};
  fn(&err, args...);
  rethrow(&err);
}

// shared_ptr whose deleter calls the C ABI free function
template <typename T, typename F>
std::shared_ptr<T> own(T* ptr, F free_fn) {
  return std::shared_ptr<T>(ptr, [free_fn](T* p) {
    if (p) {
      plaidml_error err{0, nullptr};
      free_fn(&err, p);
      if (err.msg) plaidml_string_free(err.msg);
    }
  });
}

}  // namespace ffi

inline void init() { ffi::call_void(plaidml_init); }
inline void shutdown() { ffi::call_void(plaidml_shutdown); }

enum class DType {
  INVALID = PLAIDML_DATA_INVALID,
  INTX = PLAIDML_DATA_INTX,
  UINTX = PLAIDML_DATA_UINTX,
  FLOATX = PLAIDML_DATA_FLOATX,
  BOOLEAN = PLAIDML_DATA_BOOLEAN,
  INT8 = PLAIDML_DATA_INT8,
  UINT8 = PLAIDML_DATA_UINT8,
  INT16 = PLAIDML_DATA_INT16,
  UINT16 = PLAIDML_DATA_UINT16,
  INT32 = PLAIDML_DATA_INT32,
  UINT32 = PLAIDML_DATA_UINT32,
  INT64 = PLAIDML_DATA_INT64,
  UINT64 = PLAIDML_DATA_UINT64,
  FLOAT16 = PLAIDML_DATA_FLOAT16,
  FLOAT32 = PLAIDML_DATA_FLOAT32,
  FLOAT64 = PLAIDML_DATA_FLOAT64,
  BFLOAT16 = PLAIDML_DATA_BFLOAT16,  // not in the reference: appended
  _LAST,
};

inline const char* to_string(DType dtype) {
  switch (dtype) {
    case DType::BOOLEAN: return "bool";
    case DType::INT8: return "int8";
    case DType::UINT8: return "uint8";
    case DType::INT16: return "int16";
    case DType::UINT16: return "uint16";
    case DType::INT32: return "int32";
    case DType::UINT32: return "uint32";
    case DType::INT64: return "int64";
    case DType::UINT64: return "uint64";
    case DType::FLOAT16: return "float16";
    case DType::FLOAT32: return "float32";
    case DType::FLOAT64: return "float64";
    case DType::BFLOAT16: return "bfloat16";
    default: return "<invalid>";
  }
}

class TensorShape {
 public:
  TensorShape() = default;
  TensorShape(DType dtype, const std::vector<int64_t>& sizes)
      : ptr_(ffi::own(ffi::call<plaidml_shape*>(plaidml_shape_alloc, static_cast<plaidml_datatype>(dtype), sizes.size(),
                                                sizes.data(), static_cast<const int64_t*>(nullptr)),
                      plaidml_shape_free)) {}
  TensorShape(DType dtype, const std::vector<int64_t>& sizes, const std::vector<int64_t>& strides) {
    if (sizes.size() != strides.size()) throw ffi_exception("Sizes and strides must have the same rank.");
    ptr_ = ffi::own(ffi::call<plaidml_shape*>(plaidml_shape_alloc, static_cast<plaidml_datatype>(dtype), sizes.size(),
                                              sizes.data(), strides.data()),
                    plaidml_shape_free);
  }
  explicit TensorShape(plaidml_shape* ptr) : ptr_(ffi::own(ptr, plaidml_shape_free)) {}
  explicit TensorShape(const std::shared_ptr<plaidml_shape>& ptr) : ptr_(ptr) {}

  DType dtype() const { return static_cast<DType>(ffi::call<plaidml_datatype>(plaidml_shape_get_dtype, as_ptr())); }
  size_t rank() const { return ffi::call<size_t>(plaidml_shape_get_rank, as_ptr()); }
  std::vector<int64_t> sizes() const { return integers(plaidml_shape_get_sizes); }
  std::vector<int64_t> strides() const { return integers(plaidml_shape_get_strides); }
  uint64_t byte_size() const { return ffi::call<uint64_t>(plaidml_shape_get_nbytes, as_ptr()); }
  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_shape_repr, as_ptr())); }
  bool operator==(const TensorShape& rhs) const { return str() == rhs.str(); }
  plaidml_shape* as_ptr() const { return ptr_.get(); }

 private:
  template <typename F>
  std::vector<int64_t> integers(F getter) const {
    auto ints = ffi::own(ffi::call<plaidml_integers*>(getter, as_ptr()), plaidml_integers_free);
    return std::vector<int64_t>(ints->elts, ints->elts + ints->size);
  }
  std::shared_ptr<plaidml_shape> ptr_;
};

class Buffer {
 public:
  Buffer() = default;
  // adopts caller memory: nothing is copied and nothing is owned
  Buffer(char* data, size_t size, const TensorShape& shape)
      : ptr_(ffi::own(ffi::call<plaidml_buffer*>(plaidml_buffer_adopt, shape.as_ptr(), data, size), plaidml_buffer_free)) {}
  template <typename T>
  Buffer(const std::vector<T>& vec, const TensorShape& shape)
      : ptr_(ffi::own(ffi::call<plaidml_buffer*>(plaidml_buffer_adopt, shape.as_ptr(),
                                                 reinterpret_cast<char*>(const_cast<T*>(vec.data())), vec.size() * sizeof(T)),
                      plaidml_buffer_free)) {}
  // allocates zero-filled host memory
  explicit Buffer(const TensorShape& shape)
      : ptr_(ffi::own(ffi::call<plaidml_buffer*>(plaidml_buffer_alloc, shape.as_ptr()), plaidml_buffer_free)) {}
  explicit Buffer(plaidml_buffer* ptr) : ptr_(ffi::own(ptr, plaidml_buffer_free)) {}

  char* data() { return ffi::call<char*>(plaidml_buffer_data, as_ptr()); }
  size_t size() { return ffi::call<size_t>(plaidml_buffer_size, as_ptr()); }
  TensorShape shape() { return TensorShape(ffi::call<plaidml_shape*>(plaidml_buffer_shape, as_ptr())); }
  plaidml_buffer* as_ptr() const { return ptr_.get(); }
  void copy_into(void* dst) { std::memcpy(dst, data(), size()); }
  void copy_from(const void* src) { std::memcpy(data(), src, size()); }

 private:
  std::shared_ptr<plaidml_buffer> ptr_;
};

class Program {
 public:
  explicit Program(plaidml_program* ptr) : ptr_(ffi::own(ptr, plaidml_program_free)) {}
  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_program_repr, as_ptr())); }
  // empty target: the PLAIDML_TARGET setting
  void compile(const std::string& target = "", bool debug = false) {
    ffi::call_void(plaidml_program_compile, as_ptr(), debug, target.c_str());
  }
  std::vector<TensorShape> inputs() const { return shapes(plaidml_program_get_inputs); }
  std::vector<TensorShape> outputs() const { return shapes(plaidml_program_get_outputs); }
  // (pass name, program text after the pass), in pipeline order
  std::vector<std::pair<std::string, std::string>> passes() const {
    auto kvps = ffi::own(ffi::call<plaidml_kvps*>(plaidml_program_get_passes, as_ptr()), plaidml_kvps_free);
    std::vector<std::pair<std::string, std::string>> ret;
    for (size_t i = 0; i < kvps->size; ++i) {
      // the list frees only its array (reference plaidml/core/ffi.cc:84-91): the strings are ours
      std::string key = ffi::str(kvps->elts[i].key);
      ret.emplace_back(key, ffi::str(kvps->elts[i].value));
    }
    return ret;
  }
  Buffer save(const std::unordered_map<std::string, std::string>& config = {}) const {
    std::vector<const char*> keys, values;
    for (const auto& kv : config) {
      keys.push_back(kv.first.c_str());
      values.push_back(kv.second.c_str());
    }
    return Buffer(ffi::call<plaidml_buffer*>(plaidml_program_save, as_ptr(), config.size(), keys.data(), values.data()));
  }
  plaidml_program* as_ptr() const { return ptr_.get(); }

 private:
  template <typename F>
  std::vector<TensorShape> shapes(F getter) const {
    auto list = ffi::own(ffi::call<plaidml_shapes*>(getter, as_ptr()), plaidml_shapes_free);
    std::vector<TensorShape> ret;
    // the list frees only its array (reference plaidml/core/ffi.cc:167-174): each shape handle becomes ours
    for (size_t i = 0; i < list->size; ++i) ret.emplace_back(list->elts[i]);
    return ret;
  }
  std::shared_ptr<plaidml_program> ptr_;
};

struct Settings {
  static std::string get(const std::string& key) {
    return ffi::str(ffi::call<plaidml_string*>(plaidml_settings_get, key.c_str()));
  }
  static void set(const std::string& key, const std::string& value) {
    ffi::call_void(plaidml_settings_set, key.c_str(), value.c_str());
  }
};

inline std::ostream& operator<<(std::ostream& os, const Program& x) { return os << x.str(); }
inline std::ostream& operator<<(std::ostream& os, const TensorShape& x) { return os << x.str(); }

}  // namespace plaidml

// C++ view of the execution C ABI: list_devices() and Executable, with the
// reference's names and defaults (plaidml/exec/exec.h:20-104).  An empty device
// string selects the PLAIDML_DEVICE setting (default "hip.0").
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "plaidml/core/core.h"
#include "plaidml/exec/ffi.h"

namespace plaidml {
namespace exec {

inline void init() {
  plaidml::init();
  ffi::call_void(plaidml_exec_init);
}

inline std::vector<std::string> list_devices() {
  auto strs = ffi::own(ffi::call<plaidml_strings*>(plaidml_devices_get), plaidml_strings_free);
  std::vector<std::string> ret;
  for (size_t i = 0; i < strs->size; ++i) ret.push_back(ffi::str(strs->elts[i]));
  return ret;
}

class Executable {
 public:
  explicit Executable(const Program& program, const std::string& device = "")
      : ptr_(ffi::own(ffi::call<plaidml_executable*>(plaidml_jit, program.as_ptr(), device.c_str()), plaidml_executable_free)) {}

  // Copies the inputs to the device, runs, copies the outputs back; returns the execution time in ms.
  double run(const std::vector<Buffer>& inputs, const std::vector<Buffer>& outputs) {
    std::vector<plaidml_buffer*> in, out;
    for (const Buffer& b : inputs) in.push_back(b.as_ptr());
    for (const Buffer& b : outputs) out.push_back(b.as_ptr());
    return ffi::call<double>(plaidml_executable_run, ptr_.get(), in.size(), in.data(), out.size(), out.data());
  }

 private:
  std::shared_ptr<plaidml_executable> ptr_;
};

}  // namespace exec
}  // namespace plaidml

// The `hip` runtime: device "hip.<n>" and its executables.  It fills the seam
// the reference defines with pmlc::rt::Runtime / Device / Executable
// (pmlc/rt/runtime.h:19-26, device.h:14-21, executable.h:13-25) and registers
// under the name "hip" the way `llvm_cpu` does (pmlc/rt/llvm/runtime.cc:12-35).
// An executable owns device buffers for every value of the plan, uploads
// constants and re-lays-out constant weights once when it is built (the
// reference runs its `init` closure once, pmlc/rt/jit_executable.cc:404-418),
// and on every invoke copies inputs in, launches the plan on one stream and
// copies outputs back.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "hip_plan.h"
#include "tile.h"
#include "util.h"

namespace pmlc::rt {

class Executable {
 public:
  virtual ~Executable() = default;
  // returns the wall time of the run in milliseconds, host-device transfers included
  virtual double invoke(const std::vector<util::BufferPtr>& inputs, const std::vector<util::BufferPtr>& outputs) = 0;
};

class Device {
 public:
  virtual ~Device() = default;
  virtual std::unique_ptr<Executable> compile(const std::shared_ptr<tile::Program>& program) = 0;
};

class Runtime {
 public:
  virtual ~Runtime() = default;
  virtual size_t getDeviceCount() const = 0;
  virtual std::shared_ptr<Device> getDevice(size_t ordinal) = 0;
};

// registry keyed by runtime name; device ids are "<runtime>.<ordinal>" (pmlc/rt/device_id.cc:13-38)
void registerRuntime(const std::string& id, std::shared_ptr<Runtime> runtime);
void initRuntimes();
std::vector<std::string> listDevices();
std::shared_ptr<Device> getDevice(const std::string& deviceID);

// Host memory the GPU can read and write directly (page-locked), for buffers the library allocates itself: a
// copy to or from it runs at the link's rate instead of being staged through the driver's own bounce buffers.
// Zero-initialised.  nullptr when no GPU is visible (the caller falls back to ordinary memory).
void* pinnedAlloc(size_t bytes);
void pinnedFree(void* p);

// statistics of the most recent invoke of any hip executable in this thread (for benchmarks)
struct InvokeStats {
  double kernel_ms = 0;  // first launch -> last launch, HIP events
  double h2d_ms = 0;
  double d2h_ms = 0;
  size_t launches = 0;
  double wall_ms = 0;              // the whole run, transfers included (what invoke returns)
  size_t arena_bytes = 0;          // device memory shared by the temporaries
  size_t unshared_temp_bytes = 0;  // what the temporaries would take with memory of their own
  size_t device_bytes = 0;         // arena + inputs + outputs + constants
  std::vector<double> step_ms;     // per launch, only with PLAIDML_PROFILE=1
  bool replayed = false;           // the launches ran as one recorded graph
  std::string graph_note;          // why they did not, when recording was tried and failed
};
InvokeStats lastInvokeStats();

}  // namespace pmlc::rt

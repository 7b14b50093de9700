#include "hip_runtime.h"

#include <chrono>
#include <cstring>
#include <map>
#include <regex>
#include <sstream>

#include "pml_hip.h"

namespace pmlc::rt {

using target::hip::BufferInfo;
using target::hip::Plan;
using target::hip::Step;

namespace {

thread_local InvokeStats g_stats;

void hipCheck(int status, const char* what) {
  if (status != 0) throw std::runtime_error(std::string(what) + ": " + pml_hip_last_error());
}

double nowMs() {
  using clock = std::chrono::steady_clock;
  return std::chrono::duration<double, std::milli>(clock::now().time_since_epoch()).count();
}

class HipExecutable final : public Executable {
 public:
  HipExecutable(std::shared_ptr<tile::Program> program, std::shared_ptr<Plan> plan, int ordinal)
      : program_(std::move(program)), plan_(std::move(plan)), ordinal_(ordinal) {
    hipCheck(pml_hip_init(ordinal_), "pml_hip_init");
    device_.assign(plan_->buffers.size(), nullptr);
    try {
      for (size_t i = 0; i < plan_->buffers.size(); ++i) {
        const BufferInfo& b = plan_->buffers[i];
        hipCheck(pml_hip_malloc(&device_[i], b.bytes + 16), "pml_hip_malloc");
        if (b.kind == BufferInfo::Constant)
          hipCheck(pml_hip_memcpy_h2d(device_[i], b.constant->data(), b.constant->size(), nullptr), "upload constant");
      }
      handles_.assign(plan_->steps.size(), 0);
      for (size_t i = 0; i < plan_->steps.size(); ++i) dispatch(i);
      hipCheck(pml_hip_event_create(&ev0_), "event");
      hipCheck(pml_hip_event_create(&ev1_), "event");
      hipCheck(pml_hip_stream_sync(nullptr), "sync");
    } catch (...) {
      release();
      throw;
    }
  }

  ~HipExecutable() override { release(); }

  double invoke(const std::vector<util::BufferPtr>& inputs, const std::vector<util::BufferPtr>& outputs) override {
    hipCheck(pml_hip_init(ordinal_), "pml_hip_init");
    if (inputs.size() != plan_->input_buffers.size() || outputs.size() != plan_->output_buffers.size())
      throw std::runtime_error("executable invoked with the wrong number of buffers");
    InvokeStats st;
    double t0 = nowMs();
    for (size_t i = 0; i < inputs.size(); ++i) {
      const BufferInfo& b = plan_->buffers[plan_->input_buffers[i]];
      if (inputs[i]->size() < b.bytes) throw std::runtime_error("input buffer #" + std::to_string(i) + " is too small");
      hipCheck(pml_hip_memcpy_h2d(device_[plan_->input_buffers[i]], inputs[i]->data(), b.bytes, nullptr), "h2d");
    }
    st.h2d_ms = nowMs() - t0;
    hipCheck(pml_hip_event_record(ev0_, nullptr), "event record");
    for (size_t i = 0; i < plan_->steps.size(); ++i) launch(i);
    hipCheck(pml_hip_event_record(ev1_, nullptr), "event record");
    hipCheck(pml_hip_event_sync(ev1_), "event sync");
    float ms = 0;
    hipCheck(pml_hip_event_elapsed_ms(ev0_, ev1_, &ms), "event elapsed");
    st.kernel_ms = ms;
    st.launches = plan_->steps.size();
    t0 = nowMs();
    for (size_t i = 0; i < outputs.size(); ++i) {
      const BufferInfo& b = plan_->buffers[plan_->output_buffers[i]];
      if (outputs[i]->size() < b.bytes) throw std::runtime_error("output buffer #" + std::to_string(i) + " is too small");
      hipCheck(pml_hip_memcpy_d2h(outputs[i]->data(), device_[plan_->output_buffers[i]], b.bytes, nullptr), "d2h");
    }
    st.d2h_ms = nowMs() - t0;
    g_stats = st;
    return st.kernel_ms;
  }

 private:
  std::shared_ptr<tile::Program> program_;
  std::shared_ptr<Plan> plan_;
  int ordinal_;
  std::vector<void*> device_;
  std::vector<int64_t> handles_;
  pml_hip_event ev0_ = nullptr, ev1_ = nullptr;

  void release() {
    for (int64_t h : handles_)
      if (h) pml_hip_plan_free(h);
    handles_.clear();
    for (void* p : device_)
      if (p) pml_hip_free(p);
    device_.clear();
    if (ev0_) pml_hip_event_destroy(ev0_);
    if (ev1_) pml_hip_event_destroy(ev1_);
    ev0_ = ev1_ = nullptr;
  }

  char* ptr(int buf, int64_t elem_off = 0, size_t elem_size = 1) const {
    if (buf < 0) return nullptr;
    return static_cast<char*>(device_[buf]) + elem_off * static_cast<int64_t>(elem_size);
  }

  static size_t elemSize(int dt) { return util::byteSize(static_cast<util::DataType>(dt)); }

  void dispatch(size_t i) {
    const Step& s = plan_->steps[i];
    int64_t h = 0;
    switch (s.kind) {
      case Step::Gemm: {
        h = pml_hip_gemm_dispatch(&s.gemm);
        break;
      }
      case Step::Conv2d: h = pml_hip_conv2d_dispatch(&s.conv); break;
      case Step::Dwconv2d: h = pml_hip_dwconv2d_dispatch(&s.dw); break;
      case Step::Pool2d: h = pml_hip_pool2d_dispatch(&s.pool); break;
      case Step::Eltwise: h = pml_hip_eltwise_dispatch(&s.elt); break;
      case Step::Contract: h = pml_hip_contract_dispatch(&s.con); break;
      case Step::Select:
      case Step::Index:
      case Step::Gather:
      case Step::Scatter:
      case Step::ArgSort:
      case Step::Prng:
      case Step::Copy: return;
    }
    if (!h) throw std::runtime_error("hip dispatch failed for '" + s.text + "': " + pml_hip_last_error());
    handles_[i] = h;
    // constant right-hand sides are re-laid-out once, here
    if (s.kind == Step::Gemm && s.b_constant && !s.b_is_nk)
      hipCheck(pml_hip_gemm_pack_b(h, ptr(s.b, s.b_off, elemSize(s.gemm.in_dtype)), nullptr), "pack_b");
    if (s.kind == Step::Conv2d && s.b_constant) hipCheck(pml_hip_conv2d_pack_filter(h, ptr(s.b), nullptr), "pack_filter");
  }

  void launch(size_t i) {
    const Step& s = plan_->steps[i];
    const void* operands[PML_HIP_MAX_EPI_OPERANDS] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    void* outs[PML_HIP_MAX_EPI_OPERANDS] = {nullptr, nullptr, nullptr, nullptr, nullptr, nullptr};
    for (size_t k = 0; k < s.operands.size() && k < PML_HIP_MAX_EPI_OPERANDS; ++k) operands[k] = ptr(s.operands[k]);
    for (size_t k = 0; k < s.outs.size() && k < PML_HIP_MAX_EPI_OPERANDS; ++k) outs[k] = ptr(s.outs[k]);
    switch (s.kind) {
      case Step::Gemm: {
        const size_t es = elemSize(s.gemm.in_dtype);
        const void* b = ptr(s.b, s.b_off, es);
        if (s.b_constant && !s.b_is_nk) b = nullptr;  // packed when the executable was built
        hipCheck(pml_hip_gemm_invoke(handles_[i], ptr(s.a, s.a_off, es), b, ptr(s.c, s.c_off, elemSize(s.gemm.c_dtype)),
                                     ptr(s.init), operands, outs, nullptr),
                 s.text.c_str());
        break;
      }
      case Step::Conv2d:
        hipCheck(pml_hip_conv2d_invoke(handles_[i], ptr(s.a), s.b_constant ? nullptr : ptr(s.b), ptr(s.c), ptr(s.init), operands,
                                       outs, nullptr),
                 s.text.c_str());
        break;
      case Step::Dwconv2d:
        hipCheck(pml_hip_dwconv2d_invoke(handles_[i], ptr(s.a), ptr(s.b), ptr(s.c), operands, outs, nullptr), s.text.c_str());
        break;
      case Step::Pool2d:
        hipCheck(pml_hip_pool2d_invoke(handles_[i], ptr(s.a), ptr(s.c), ptr(s.out2), nullptr), s.text.c_str());
        break;
      case Step::Eltwise:
        hipCheck(pml_hip_eltwise_invoke(handles_[i], ptr(s.a), ptr(s.c), operands, outs, nullptr), s.text.c_str());
        break;
      case Step::Select:
        hipCheck(pml_hip_select(&s.sel, operands[0], operands[1], operands[2], ptr(s.c), nullptr), s.text.c_str());
        break;
      case Step::Index:
        hipCheck(pml_hip_index(ptr(s.c), static_cast<int32_t>(s.index_sizes.size()), s.index_sizes.data(), s.index_axis, nullptr),
                 s.text.c_str());
        break;
      case Step::Contract:
        hipCheck(pml_hip_contract_invoke(handles_[i], operands, ptr(s.c), nullptr), s.text.c_str());
        break;
      case Step::Copy:
        hipCheck(pml_hip_memcpy_d2d(ptr(s.c), ptr(s.a), s.copy_bytes, nullptr), s.text.c_str());
        break;
      case Step::Gather:
        hipCheck(pml_hip_gather(&s.gat, operands[0], operands[1], ptr(s.c), nullptr), s.text.c_str());
        break;
      case Step::Scatter:
        hipCheck(pml_hip_scatter(&s.sca, operands[0], operands[1], operands[2], ptr(s.c), nullptr), s.text.c_str());
        break;
      case Step::ArgSort:
        hipCheck(pml_hip_argsort(&s.srt, operands[0], ptr(s.c), nullptr), s.text.c_str());
        break;
      case Step::Prng:
        hipCheck(pml_hip_prng(operands[0], s.prng_count, s.prng_state ? nullptr : ptr(s.c), s.prng_state ? ptr(s.c) : nullptr, nullptr),
                 s.text.c_str());
        break;
    }
  }
};

class HipDevice final : public Device {
 public:
  explicit HipDevice(int ordinal) : ordinal_(ordinal) {}
  std::unique_ptr<Executable> compile(const std::shared_ptr<tile::Program>& program) final {
    if (!program->compiled || program->target != "hip")
      throw std::runtime_error("the program was not compiled for target 'hip'");
    auto plan = std::static_pointer_cast<Plan>(program->compiled);
    return std::make_unique<HipExecutable>(program, plan, ordinal_);
  }

 private:
  int ordinal_;
};

class HipRuntime final : public Runtime {
 public:
  HipRuntime() {
    count_ = static_cast<size_t>(pml_hip_device_count());
    if (count_ == 0) throw std::runtime_error("no HIP device is visible");
  }
  size_t getDeviceCount() const final { return count_; }
  std::shared_ptr<Device> getDevice(size_t ordinal) final {
    if (ordinal >= count_) throw std::out_of_range("hip device ordinal out of range");
    return std::make_shared<HipDevice>(static_cast<int>(ordinal));
  }

 private:
  size_t count_ = 0;
};

std::map<std::string, std::shared_ptr<Runtime>>& registry() {
  static std::map<std::string, std::shared_ptr<Runtime>> r;
  return r;
}

}  // namespace

InvokeStats lastInvokeStats() { return g_stats; }

void registerRuntime(const std::string& id, std::shared_ptr<Runtime> runtime) {
  if (registry().count(id)) throw std::runtime_error("Multiple runtime registrations for id: " + id);
  registry()[id] = std::move(runtime);
}

void initRuntimes() {
  static bool done = false;
  if (done) return;
  done = true;
  // a runtime whose construction fails (no GPU) is skipped, as the reference skips a throwing factory
  // (pmlc/rt/runtime_registry.cc:48-59)
  try {
    registerRuntime("hip", std::make_shared<HipRuntime>());
  } catch (const std::exception&) {
  }
}

std::vector<std::string> listDevices() {
  std::vector<std::string> out;
  for (const auto& kv : registry())
    for (size_t i = 0; i < kv.second->getDeviceCount(); ++i) out.push_back(kv.first + "." + std::to_string(i));
  return out;
}

std::shared_ptr<Device> getDevice(const std::string& deviceID) {
  static const std::regex re("([[:alpha:]][_[:alnum:]]*(?:-[[:alpha:]][_[:alnum:]]*)*)\\.([[:digit:]]+)");
  std::smatch m;
  if (!std::regex_match(deviceID, m, re)) throw std::runtime_error("Invalid device name: " + deviceID);
  auto it = registry().find(m[1].str());
  if (it == registry().end()) throw std::runtime_error("Unable to find " + m[1].str() + " runtime");
  return it->second->getDevice(std::stoul(m[2].str()));
}

}  // namespace pmlc::rt

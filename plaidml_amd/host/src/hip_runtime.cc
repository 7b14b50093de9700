#include "hip_runtime.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <regex>
#include <sstream>

#include "pml_hip.h"

namespace pmlc::rt {

using target::hip::BufferInfo;
using target::hip::Plan;
using target::hip::Step;

namespace {

thread_local InvokeStats g_stats;

constexpr size_t kAlign = 256;  // arena offsets; also the slack behind every value (kernels read whole 16-byte vectors)
size_t padded(size_t bytes) { return (bytes + 16 + kAlign - 1) / kAlign * kAlign; }

bool profileRequested() {
  const char* e = std::getenv("PLAIDML_PROFILE");
  return e && std::string(e) == "1";
}

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
    owned_.assign(plan_->buffers.size(), false);
    try {
      // Inputs, outputs and constants keep memory of their own for the life of the executable; temporaries
      // share one arena, each placed by the span of steps in which it is live (what the reference's
      // resize-tmps / dealloc placement does for its heap temporaries, pmlc/target/x86/pipeline.cc:289-360).
      const std::vector<size_t> offsets = placeTemporaries();
      if (arena_bytes_) hipCheck(pml_hip_malloc(&arena_, arena_bytes_), "pml_hip_malloc (arena)");
      for (size_t i = 0; i < plan_->buffers.size(); ++i) {
        const BufferInfo& b = plan_->buffers[i];
        if (b.kind == BufferInfo::Temp) {
          device_[i] = static_cast<char*>(arena_) + offsets[i];
          continue;
        }
        hipCheck(pml_hip_malloc(&device_[i], b.bytes + 16), "pml_hip_malloc");
        owned_[i] = true;
        fixed_bytes_ += padded(b.bytes);
        if (b.kind == BufferInfo::Constant)
          hipCheck(pml_hip_memcpy_h2d(device_[i], b.constant->data(), b.constant->size(), nullptr), "upload constant");
      }
      handles_.assign(plan_->steps.size(), 0);
      for (size_t i = 0; i < plan_->steps.size(); ++i) dispatch(i);
      hipCheck(pml_hip_event_create(&ev0_), "event");
      hipCheck(pml_hip_event_create(&ev1_), "event");
      hipCheck(pml_hip_stream_create(&stream_), "stream");
      hipCheck(pml_hip_stream_sync(nullptr), "sync");
      // Recording is for runs of plain kernel launches and device-to-device copies: the sort, scatter, gather, index and random-number steps keep
      // state or sizes on the host side of their entry points and stay with one-by-one launches.
      graphable_ = plan_->graph && plan_->steps.size() > 1;
      for (const Step& s : plan_->steps)
        if (s.kind != Step::Gemm && s.kind != Step::Conv2d && s.kind != Step::Dwconv2d && s.kind != Step::Pool2d &&
            s.kind != Step::Eltwise && s.kind != Step::Contract && s.kind != Step::Select && s.kind != Step::Copy &&
            s.kind != Step::Softmax)
          graphable_ = false;
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
    const double start = nowMs();
    double t0 = start;
    const bool profile = profileRequested();
    for (size_t i = 0; i < inputs.size(); ++i) {
      const BufferInfo& b = plan_->buffers[plan_->input_buffers[i]];
      if (inputs[i]->size() < b.bytes) throw std::runtime_error("input buffer #" + std::to_string(i) + " is too small");
      hipCheck(pml_hip_memcpy_h2d(device_[plan_->input_buffers[i]], inputs[i]->data(), b.bytes, stream_), "h2d");
    }
    st.h2d_ms = nowMs() - t0;
    if (profile && step_events_.size() != plan_->steps.size() + 1) {
      step_events_.assign(plan_->steps.size() + 1, nullptr);
      for (auto& e : step_events_) hipCheck(pml_hip_event_create(&e), "event");
    }
    // The launches of a run never change (same plans, same device buffers), so from the third run on they are
    // replayed as one graph recorded during that run; the first two run one by one (first runs of a kernel plan may
    // allocate, which cannot be recorded).  A recording that fails leaves the executable with one-by-one launches.
    if (graphable_ && !profile && !graph_ && runs_ >= 2) record();
    ++runs_;
    hipCheck(pml_hip_event_record(ev0_, stream_), "event record");
    if (graph_ && !profile) {
      hipCheck(pml_hip_graph_launch(graph_, stream_), "graph launch");
      st.replayed = true;
    } else {
      for (size_t i = 0; i < plan_->steps.size(); ++i) {
        if (profile) hipCheck(pml_hip_event_record(step_events_[i], stream_), "event record");
        launch(i);
      }
    }
    if (profile) hipCheck(pml_hip_event_record(step_events_.back(), stream_), "event record");
    hipCheck(pml_hip_event_record(ev1_, stream_), "event record");
    hipCheck(pml_hip_event_sync(ev1_), "event sync");
    float ms = 0;
    hipCheck(pml_hip_event_elapsed_ms(ev0_, ev1_, &ms), "event elapsed");
    st.kernel_ms = ms;
    st.launches = plan_->steps.size();
    st.graph_note = graph_note_;
    st.arena_bytes = arena_bytes_;
    st.unshared_temp_bytes = unshared_temp_bytes_;
    st.device_bytes = arena_bytes_ + fixed_bytes_;
    if (profile) {
      // One row per launch, in the reference's format (pmlc/rt/instrument.cc:22-43: id, loc, tag, seconds since
      // the previous point, seconds since the start); loc is the plan's line for the step, tag its kind.
      std::printf("\"id\",\"loc\",\"tag\",\"elapsed\",\"accumulated\"\n");
      double total = 0;
      st.step_ms.resize(plan_->steps.size());
      for (size_t i = 0; i < plan_->steps.size(); ++i) {
        float step = 0;
        hipCheck(pml_hip_event_elapsed_ms(step_events_[i], step_events_[i + 1], &step), "event elapsed");
        st.step_ms[i] = step;
        total += step;
        std::printf("%03d,\"%s\",%d,%7.6f,%7.6f\n", static_cast<int>(i), plan_->steps[i].text.c_str(),
                    static_cast<int>(plan_->steps[i].kind), step * 1e-3, total * 1e-3);
      }
      std::printf("%03d,%s,%d,%7.6f,%7.6f\n", 9999, "endTime", 9999, 0.0, total * 1e-3);
      std::fflush(stdout);
    }
    t0 = nowMs();
    for (size_t i = 0; i < outputs.size(); ++i) {
      const BufferInfo& b = plan_->buffers[plan_->output_buffers[i]];
      if (outputs[i]->size() < b.bytes) throw std::runtime_error("output buffer #" + std::to_string(i) + " is too small");
      hipCheck(pml_hip_memcpy_d2h(outputs[i]->data(), device_[plan_->output_buffers[i]], b.bytes, stream_), "d2h");
    }
    st.d2h_ms = nowMs() - t0;
    st.wall_ms = nowMs() - start;
    g_stats = st;
    // wall time of the whole run, transfers included, as the reference returns the time around its jitted main
    // (pmlc/rt/jit_executable.cc:484-490); the device time alone is in the statistics
    return st.wall_ms;
  }

 private:
  std::shared_ptr<tile::Program> program_;
  std::shared_ptr<Plan> plan_;
  int ordinal_;
  std::vector<void*> device_;
  std::vector<bool> owned_;
  void* arena_ = nullptr;
  size_t arena_bytes_ = 0, fixed_bytes_ = 0, unshared_temp_bytes_ = 0;
  std::vector<int64_t> handles_;
  pml_hip_event ev0_ = nullptr, ev1_ = nullptr;
  std::vector<pml_hip_event> step_events_;
  pml_hip_stream stream_ = nullptr;  // every copy and launch of this executable
  pml_hip_graph graph_ = nullptr;    // the launches of one run, recorded
  bool graphable_ = false;
  int runs_ = 0;
  std::string graph_note_;

  void record() {
    if (pml_hip_capture_begin(stream_) != 0) {
      graph_note_ = pml_hip_last_error();
      graphable_ = false;
      return;
    }
    bool ok = true;
    try {
      for (size_t i = 0; i < plan_->steps.size(); ++i) launch(i);
    } catch (const std::exception& e) {
      graph_note_ = e.what();
      ok = false;
    }
    pml_hip_graph g = nullptr;
    if (pml_hip_capture_end(stream_, &g) != 0 || !ok) {
      if (ok) graph_note_ = pml_hip_last_error();
      if (g) pml_hip_graph_destroy(g);
      graphable_ = false;
      return;
    }
    graph_ = g;
  }

  // Offsets of the temporaries in the arena.  A temporary is live from the first to the last step that names
  // it; steps run in order on one stream, so two temporaries whose spans do not overlap may share bytes.  A
  // value freed by step i is not handed to a value that step i itself defines (kernels read while they write).
  std::vector<size_t> placeTemporaries() {
    const size_t nb = plan_->buffers.size(), ns = plan_->steps.size();
    std::vector<int> first(nb, -1), last(nb, -1);
    auto touch = [&](int buf, size_t step) {
      if (buf < 0 || static_cast<size_t>(buf) >= nb) return;
      if (first[buf] < 0) first[buf] = static_cast<int>(step);
      last[buf] = static_cast<int>(step);
    };
    for (size_t i = 0; i < ns; ++i) {
      const Step& s = plan_->steps[i];
      for (int b : {s.a, s.b, s.c, s.init, s.out2, s.a2, s.b2, s.init2}) touch(b, i);
      for (int b : s.operands) touch(b, i);
      for (int b : s.outs) touch(b, i);
    }
    std::vector<size_t> offsets(nb, 0);
    struct Block { size_t off, size; };
    std::vector<Block> free_blocks;
    std::vector<std::vector<int>> starts(ns + 1), ends(ns + 1);
    for (size_t b = 0; b < nb; ++b) {
      if (plan_->buffers[b].kind != BufferInfo::Temp) continue;
      if (first[b] < 0) continue;  // a value no launch touches (its producer was fused away) takes no memory
      unshared_temp_bytes_ += padded(plan_->buffers[b].bytes);
      const size_t f = first[b] < 0 ? 0 : static_cast<size_t>(first[b]);
      const size_t l = last[b] < 0 ? 0 : static_cast<size_t>(last[b]);
      starts[f].push_back(static_cast<int>(b));
      ends[l].push_back(static_cast<int>(b));
    }
    auto release_block = [&](size_t off, size_t size) {
      free_blocks.push_back({off, size});
      std::sort(free_blocks.begin(), free_blocks.end(), [](const Block& x, const Block& y) { return x.off < y.off; });
      for (size_t k = 0; k + 1 < free_blocks.size();) {
        if (free_blocks[k].off + free_blocks[k].size == free_blocks[k + 1].off) {
          free_blocks[k].size += free_blocks[k + 1].size;
          free_blocks.erase(free_blocks.begin() + static_cast<long>(k) + 1);
        } else {
          ++k;
        }
      }
    };
    for (size_t i = 0; i <= ns; ++i) {
      // larger values first: they are the hard ones to place
      std::sort(starts[i].begin(), starts[i].end(),
                [&](int x, int y) { return plan_->buffers[x].bytes > plan_->buffers[y].bytes; });
      for (int b : starts[i]) {
        const size_t need = padded(plan_->buffers[b].bytes);
        size_t best = free_blocks.size();
        for (size_t k = 0; k < free_blocks.size(); ++k)
          if (free_blocks[k].size >= need && (best == free_blocks.size() || free_blocks[k].size < free_blocks[best].size)) best = k;
        if (best < free_blocks.size()) {
          offsets[b] = free_blocks[best].off;
          free_blocks[best].off += need;
          free_blocks[best].size -= need;
          if (!free_blocks[best].size) free_blocks.erase(free_blocks.begin() + static_cast<long>(best));
        } else if (!free_blocks.empty() && free_blocks.back().off + free_blocks.back().size == arena_bytes_) {
          // grow the free block at the end of the arena
          offsets[b] = free_blocks.back().off;
          arena_bytes_ = offsets[b] + need;
          free_blocks.pop_back();
        } else {
          offsets[b] = arena_bytes_;
          arena_bytes_ += need;
        }
      }
      for (int b : ends[i]) release_block(offsets[b], padded(plan_->buffers[b].bytes));
    }
    return offsets;
  }

  void release() {
    for (int64_t h : handles_)
      if (h) pml_hip_plan_free(h);
    handles_.clear();
    for (size_t i = 0; i < device_.size(); ++i)
      if (device_[i] && owned_[i]) pml_hip_free(device_[i]);
    device_.clear();
    if (arena_) pml_hip_free(arena_);
    arena_ = nullptr;
    for (auto& e : step_events_)
      if (e) pml_hip_event_destroy(e);
    step_events_.clear();
    if (ev0_) pml_hip_event_destroy(ev0_);
    if (ev1_) pml_hip_event_destroy(ev1_);
    ev0_ = ev1_ = nullptr;
    if (graph_) pml_hip_graph_destroy(graph_);
    graph_ = nullptr;
    if (stream_) pml_hip_stream_destroy(stream_);
    stream_ = nullptr;
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
      case Step::Softmax:
      case Step::Copy: return;
    }
    if (!h) throw std::runtime_error("hip dispatch failed for '" + s.text + "': " + pml_hip_last_error());
    handles_[i] = h;
    // constant right-hand sides are re-laid-out once, here
    if (s.kind == Step::Gemm && s.b_constant && !s.b_is_nk)
      hipCheck(pml_hip_gemm_pack_b(h, ptr(s.b, s.b_off, elemSize(s.gemm.in_dtype)), nullptr), "pack_b");
    if (s.kind == Step::Gemm && s.gemm.k2 > 0 && s.b2_constant && !s.b_is_nk)
      hipCheck(pml_hip_gemm_pack_b2(h, ptr(s.b2, s.b2_off, elemSize(s.gemm.in_dtype)), nullptr), "pack_b2");
    if (s.kind == Step::Conv2d && s.b_constant) hipCheck(pml_hip_conv2d_pack_filter(h, ptr(s.b), nullptr), "pack_filter");
    if (s.kind == Step::Dwconv2d && s.b_constant) hipCheck(pml_hip_dwconv2d_pack_filter(h, ptr(s.b), nullptr), "pack_filter");
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
        if (s.gemm.k2 > 0) {
          const void* b2 = ptr(s.b2, s.b2_off, es);
          if (s.b2_constant && !s.b_is_nk) b2 = nullptr;
          hipCheck(pml_hip_gemm_invoke2(handles_[i], ptr(s.a, s.a_off, es), b, ptr(s.c, s.c_off, elemSize(s.gemm.c_dtype)), ptr(s.init),
                                        ptr(s.a2, s.a2_off, es), b2, ptr(s.init2), operands, outs, stream_),
                   s.text.c_str());
          break;
        }
        hipCheck(pml_hip_gemm_invoke(handles_[i], ptr(s.a, s.a_off, es), b, ptr(s.c, s.c_off, elemSize(s.gemm.c_dtype)),
                                     ptr(s.init), operands, outs, stream_),
                 s.text.c_str());
        break;
      }
      case Step::Conv2d:
        hipCheck(pml_hip_conv2d_invoke(handles_[i], ptr(s.a), s.b_constant ? nullptr : ptr(s.b), ptr(s.c), ptr(s.init), operands,
                                       outs, stream_),
                 s.text.c_str());
        break;
      case Step::Dwconv2d:
        hipCheck(pml_hip_dwconv2d_invoke(handles_[i], ptr(s.a), s.b_constant ? nullptr : ptr(s.b), ptr(s.c), operands, outs, stream_),
                 s.text.c_str());
        break;
      case Step::Pool2d:
        hipCheck(pml_hip_pool2d_invoke(handles_[i], ptr(s.a), ptr(s.c), ptr(s.out2), stream_), s.text.c_str());
        break;
      case Step::Eltwise:
        hipCheck(pml_hip_eltwise_invoke(handles_[i], ptr(s.a), ptr(s.c), operands, outs, stream_), s.text.c_str());
        break;
      case Step::Select:
        hipCheck(pml_hip_select(&s.sel, operands[0], operands[1], operands[2], ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::Softmax:
        hipCheck(pml_hip_softmax(&s.sm, ptr(s.a), ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::Index:
        hipCheck(pml_hip_index(ptr(s.c), static_cast<int32_t>(s.index_sizes.size()), s.index_sizes.data(), s.index_axis, stream_),
                 s.text.c_str());
        break;
      case Step::Contract:
        hipCheck(pml_hip_contract_invoke(handles_[i], operands, ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::Copy:
        hipCheck(pml_hip_memcpy_d2d(ptr(s.c), ptr(s.a), s.copy_bytes, stream_), s.text.c_str());
        break;
      case Step::Gather:
        hipCheck(pml_hip_gather(&s.gat, operands[0], operands[1], ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::Scatter:
        hipCheck(pml_hip_scatter(&s.sca, operands[0], operands[1], operands[2], ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::ArgSort:
        hipCheck(pml_hip_argsort(&s.srt, operands[0], ptr(s.c), stream_), s.text.c_str());
        break;
      case Step::Prng:
        hipCheck(pml_hip_prng(operands[0], s.prng_count, s.prng_state ? nullptr : ptr(s.c), s.prng_state ? ptr(s.c) : nullptr, stream_),
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

// Page-locked host memory for buffers the library allocates itself.  Asking for it initialises the GPU runtime as a
// side effect, so a process that must not touch the GPU (one that only builds programs, or that will exec another
// program) sets PLAIDML_PINNED=0; the total is capped (PLAIDML_PINNED_MAX_MB, default 4096) because page-locked
// memory is taken from what the host can page.  Beyond the cap, and on any failure, the caller falls back to
// ordinary memory (nullptr here).
namespace {
std::mutex g_pinned_mutex;
std::map<void*, size_t> g_pinned_sizes;
size_t g_pinned_total = 0;
}  // namespace

void* pinnedAlloc(size_t bytes) {
  const std::string enabled = util::Settings::Instance()->get("PLAIDML_PINNED");
  if (enabled == "0" || enabled == "false" || enabled == "off") return nullptr;
  const std::string cap_text = util::Settings::Instance()->get("PLAIDML_PINNED_MAX_MB");
  const size_t cap = (cap_text.empty() ? size_t{4096} : static_cast<size_t>(std::strtoull(cap_text.c_str(), nullptr, 10))) << 20;
  {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    if (bytes > cap || g_pinned_total > cap - bytes) return nullptr;
  }
  initRuntimes();
  if (listDevices().empty()) return nullptr;
  void* p = nullptr;
  if (pml_hip_host_alloc(&p, bytes) != 0 || !p) return nullptr;
  std::memset(p, 0, bytes);
  std::lock_guard<std::mutex> lock(g_pinned_mutex);
  g_pinned_sizes[p] = bytes;
  g_pinned_total += bytes;
  return p;
}

void pinnedFree(void* p) {
  if (!p) return;
  {
    std::lock_guard<std::mutex> lock(g_pinned_mutex);
    const auto it = g_pinned_sizes.find(p);
    if (it != g_pinned_sizes.end()) {
      g_pinned_total -= it->second;
      g_pinned_sizes.erase(it);
    }
  }
  pml_hip_host_free(p);
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

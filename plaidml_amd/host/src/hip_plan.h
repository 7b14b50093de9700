// The `hip` target: turns a Tile program into a kernel plan for the gfx950 kernel
// library.  It stands where the reference's `llvm_cpu` target pipeline stands
// (pmlc/target/x86/pipeline.cc:259-402) but does not lower through loops: each
// contraction is classified by the strides of its accesses (the idea of the
// reference GEMM stencil, pmlc/dialect/pxa/transforms/stencil_gemm.cc:297-321),
// its single-use elementwise consumers are folded into the kernel's tail (the
// role of pxa-fusion and x86-tpp-combine, pmlc/target/x86/tpp_combine.cc:30-140),
// and the result is a list of launches.  Building a plan needs no device.
#pragma once

#include <memory>
#include <string>
#include <vector>

#include "pml_hip.h"
#include "tile.h"

namespace pmlc::target::hip {

struct BufferInfo {
  enum Kind { Input, Output, Constant, Temp } kind = Temp;
  int index = 0;                 // Input / Output: position in the program signature
  size_t bytes = 0;
  util::BufferPtr constant;      // Constant: host bytes uploaded once when the executable is built
  std::string name;
};

struct Step {
  enum Kind { Gemm, Conv2d, Dwconv2d, Pool2d, Eltwise, Select, Index, Contract, Copy, Gather, Scatter, ArgSort, Prng, Softmax } kind = Copy;
  std::string text;  // one line for the plan dump
  std::string schedule;  // "{tile=...,conv=...}" when the target options or a schedule file named this step's tiling
  // descriptors (only the one matching `kind` is meaningful)
  pml_hip_gemm_desc gemm{};
  pml_hip_conv2d_desc conv{};
  pml_hip_dwconv2d_desc dw{};
  pml_hip_pool2d_desc pool{};
  pml_hip_eltwise_desc elt{};
  pml_hip_select_desc sel{};
  pml_hip_contract_desc con{};
  pml_hip_gather_desc gat{};
  pml_hip_scatter_desc sca{};
  pml_hip_argsort_desc srt{};
  pml_hip_softmax_desc sm{};
  int64_t prng_count = 0;   // Prng: values drawn
  bool prng_state = false;  //       the step yields the advanced state instead of the values
  int index_axis = 0;
  std::vector<int64_t> index_sizes;
  // buffer ids (-1 = none) and element offsets applied to the base pointers
  int a = -1, b = -1, c = -1, init = -1, out2 = -1;
  int64_t a_off = 0, b_off = 0, c_off = 0, init_off = 0;
  // Gemm with a second product (gemm.k2 > 0): its left- and right-hand side and per-column initial value
  int a2 = -1, b2 = -1, init2 = -1;
  int64_t a2_off = 0, b2_off = 0;
  bool b2_constant = false;
  std::vector<int> operands;       // tail operands / contraction sources / select inputs
  std::vector<int64_t> operand_off;
  std::vector<int> outs;           // extra outputs of STORE steps (index = STORE's operand field)
  bool b_is_nk = false;            // Gemm: right-hand side is already [N][K]
  bool b_constant = false;         // Gemm / Conv2d / Dwconv2d: right-hand side / filter is a program constant (pack once)
  size_t copy_bytes = 0;           // Copy
  // roofline bookkeeping for reports
  double flops = 0;
  double bytes = 0;
};

struct Plan {
  std::vector<BufferInfo> buffers;
  std::vector<Step> steps;
  std::vector<int> input_buffers;   // buffer id per program input
  std::vector<int> output_buffers;  // buffer id per program output
  bool graph = true;                // the runtime may replay the launches of a run as one recorded graph
  std::string dump() const;
};

struct Options {
  bool fuse = true;        // fold elementwise consumers into kernel tails
  bool specialise = true;  // use the MFMA / window kernels; false = every contraction through the general kernel
  // fp32 GEMMs and convolutions on the bf16 matrix cores, every operand value split into a bf16 head and a bf16
  // remainder (three products per term, about 2^-16 relative error per product): `hip{fp32=bf16x3}`
  bool fp32_as_bf16x3 = false;
  // Schedule overrides (the reference: PLAIDML_SCHEDULE_PATH, pmlc/target/x86/pipeline.cc:267-272).  `tile` / `conv`
  // (`hip{tile=128x128w8,conv=igemm}`) apply to every matrix product / convolution of the program; `schedule_path` names
  // a file of plan-dump lines, "[n] <step text> {tile=...,conv=...}", that apply to the steps whose text they repeat --
  // a plan dump edited by hand is such a file.  Names: pml_hip_tile_name, and igemm / patches / ldsfilter / blocks.
  std::string tile, conv, schedule_path;
  // `hip{graph=0}`: every run launches its kernels one by one (the default records the launches of the third run of an
  // executable into a HIP graph and replays that from then on: at batch 1 the launches cost more than the kernels)
  bool graph = true;
};

// Runs the pipeline on a copy of the program's op list and returns the plan.
std::shared_ptr<Plan> buildPlan(tile::Program* program, const Options& options);

}  // namespace pmlc::target::hip

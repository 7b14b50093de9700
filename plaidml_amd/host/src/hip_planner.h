// The planner behind buildPlan (hip_plan.h), shared by the translation units that hold its parts:
//   hip_plan.cc        the driver: buffers, the walk over the program, schedule overrides, the plan dump
//   hip_plan_match.cc  recognising matrix products, convolutions, depthwise convolutions and pooling in a contraction
//   hip_plan_fuse.cc   elementwise tails folded into kernels, second products, row pitches, dead steps
//   hip_plan_emit.cc   elementwise and special operations, and the general loop nest for every other contraction
// Not part of the library's interface.
#pragma once

#include <algorithm>
#include <array>
#include <cstring>
#include <fstream>
#include <map>
#include <numeric>
#include <set>
#include <sstream>

#include "hip_plan.h"

namespace pmlc::target::hip {

using tile::Affine;
using tile::AggKind;
using tile::ComboKind;
using tile::Op;
using tile::Program;
using tile::Value;
using tile::ValuePtr;
using util::DataType;
using util::TensorShape;

inline int hipType(DataType dt) { return static_cast<int>(dt); }  // the kernel library uses plaidml_datatype values

inline int hipAgg(AggKind a) {
  switch (a) {
    case AggKind::assign: return PML_HIP_AGG_ASSIGN;
    case AggKind::add: return PML_HIP_AGG_ADD;
    case AggKind::max: return PML_HIP_AGG_MAX;
    case AggKind::min: return PML_HIP_AGG_MIN;
    case AggKind::mul: return PML_HIP_AGG_MUL;
  }
  return 0;
}
inline int hipCombo(ComboKind c) {
  switch (c) {
    case ComboKind::none: return PML_HIP_COMBO_NONE;
    case ComboKind::add: return PML_HIP_COMBO_ADD;
    case ComboKind::cond: return PML_HIP_COMBO_COND;
    case ComboKind::eq: return PML_HIP_COMBO_EQ;
    case ComboKind::mul: return PML_HIP_COMBO_MUL;
  }
  return 0;
}

inline bool is64(DataType dt) { return util::byteSize(dt) == 8; }

// A contraction with its range-1 indices folded into the constants.
struct Normalised {
  size_t nIdx = 0;
  std::vector<bool> active;
  std::vector<std::vector<Affine>> acc;  // [0] sink, [1..] sources
  std::vector<tile::ConstraintForm> cons;
};

inline Normalised normalise(const Op& op) {
  Normalised n;
  n.nIdx = op.idxNames.size();
  n.active.resize(n.nIdx);
  for (size_t v = 0; v < n.nIdx; ++v) n.active[v] = op.lower[v] < op.upper[v];
  auto fold = [&](Affine a) {
    for (size_t v = 0; v < n.nIdx; ++v) {
      if (!n.active[v] && a.coef[v]) {
        a.c0 += a.coef[v] * op.lower[v];
        a.coef[v] = 0;
      }
    }
    return a;
  };
  for (const auto& forms : op.accesses) {
    std::vector<Affine> out;
    for (const Affine& a : forms) out.push_back(fold(a));
    n.acc.push_back(out);
  }
  for (const auto& c : op.constraints) {
    tile::ConstraintForm cf;
    cf.lhs = fold(c.lhs);
    cf.rhs = c.rhs;
    n.cons.push_back(cf);
  }
  return n;
}

// min / max of a form over the box
inline void formRange(const Op& op, const Affine& a, int64_t* lo, int64_t* hi) {
  int64_t l = a.c0, h = a.c0;
  for (size_t v = 0; v < a.coef.size(); ++v) {
    const int64_t c = a.coef[v];
    if (!c) continue;
    const int64_t x = c * op.lower[v], y = c * op.upper[v];
    l += std::min(x, y);
    h += std::max(x, y);
  }
  *lo = l;
  *hi = h;
}

// true when the box alone guarantees 0 <= a < size with a integral
inline bool impliedByBox(const Op& op, const Affine& a, int64_t size) {
  if (a.den != 1) return false;
  int64_t lo, hi;
  formRange(op, a, &lo, &hi);
  return lo >= 0 && hi < size;
}

inline bool emptyBox(const Op& op) {
  for (size_t v = 0; v < op.lower.size(); ++v)
    if (op.lower[v] > op.upper[v]) return true;
  return false;
}

// flat element stride of every index in one access (plain multiples only); false if a form has den != 1
inline bool indexStrides(const std::vector<Affine>& forms, const TensorShape& shape, std::vector<int64_t>* strides,
                  int64_t* base) {
  const auto dense = shape.denseStrides();
  const size_t n = forms.empty() ? 0 : forms[0].coef.size();
  strides->assign(n, 0);
  *base = 0;
  for (size_t d = 0; d < forms.size(); ++d) {
    if (forms[d].den != 1) return false;
    for (size_t v = 0; v < n; ++v) (*strides)[v] += forms[d].coef[v] * dense[d];
    *base += forms[d].c0 * dense[d];
  }
  return true;
}

struct TailBuild {
  pml_hip_epilogue tail{};
  std::vector<int> operand_bufs;
  std::vector<int64_t> operand_offs;
  std::vector<std::array<int64_t, PML_HIP_MAX_RANK>> nd_strides;
  std::vector<int> outs;
  ValuePtr final_value;
  DataType final_dtype = DataType::invalid;
  std::vector<size_t> consumed;
};

class Planner {
 public:
  Planner(Program* program, const Options& options) : prog_(program), opt_(options), plan_(std::make_shared<Plan>()) {
    plan_->graph = options.graph;
  }

  std::shared_ptr<Plan> run();
  static int convPathByName(const std::string& name);
  static int tileByName(const std::string& name);
  struct Rule {
    int tile = -1, conv = 0;
  };
  static Rule parseRule(const std::string& text);
  void applySchedule();
  void fuseSecondProducts();
  void padDepthwiseResults();
  void fusePoolIntoConv();
  void pruneDeadSteps();

 private:
  Program* prog_;
  Options opt_;
  std::shared_ptr<Plan> plan_;
  std::map<const Value*, int> bufferOf_;
  std::map<const Value*, std::vector<size_t>> users_;
  std::map<const Value*, size_t> producer_;
  std::set<const Value*> outputs_;
  std::set<size_t> consumed_;
  void analyse();
  void rewriteSelectMinMax();
  int newBuffer(BufferInfo::Kind kind, size_t bytes, const std::string& name);
  int bufferFor(const ValuePtr& v);
  int scalarConstant(DataType dt, double f, int64_t i);

  // ----- elementwise chains -------------------------------------------------------------

  static int unaryOpcode(const std::string& fn);
  static void checkStepType(const std::string& fn, DataType dt);
  // comparisons and truth-value operations compute in their operands' promoted type and yield i1
  static bool computesInOperandType(const std::string& fn) { return ast::isCompareOp(fn) || ast::isLogicalOp(fn); }
  static int binaryOpcode(const std::string& fn, bool running_first);
  static bool ndStrides(const TensorShape& shape, const TensorShape& out, std::array<int64_t, PML_HIP_MAX_RANK>* st);
  static bool rowColStrides(const TensorShape& shape, const TensorShape& out, int64_t* rs, int64_t* cs);
  void extendTail(TailBuild* tb, ValuePtr value, size_t root, bool two_d, bool allow64);
  static std::string tailText(const TailBuild& tb);
  void attachTail(Step* s, const TailBuild& tb);

  // ----- emission -------------------------------------------------------------------------

  void emit(size_t i);
  void emitSpecial(size_t i);
  void emitEltwise(size_t i);
  const Op* castProducer(const ValuePtr& v, DataType from);
  void emitContraction(size_t i);
  bool denseInit(const Op& op, int32_t* kind, int32_t* dtype, int64_t* rs, int64_t* cs, int* buf);
  bool denseTypes(const Op& op, ValuePtr* a, ValuePtr* b, int* in_dt, int* out_dt);
  bool tryGemm(size_t i);
  bool unconsume(const TailBuild& tb);

  // spatial form s*x + d*k - p: finds the output index (coef s) and tap index (coef d)
  struct Spatial {
    int out_idx = -1, tap_idx = -1;
    int64_t stride = 1, dil = 1, pad = 0;
  };
  bool spatialForm(const Affine& a, const std::vector<bool>& in_out, const std::vector<bool>& active, Spatial* sp);
  bool windowOutput(const Op& op, const Normalised& n, const TensorShape& os, int oi[4], std::vector<bool>* in_out);
  // the access form is the index idx, or the constant 0 where that index was folded away (idx < 0)
  static bool sameIndex(const Affine& a, int idx) { return idx >= 0 ? a.plainIndex() == idx : (a.isConstant() && a.c0 == 0); }

  bool tryConv(size_t i);
  bool tryDepthwise(size_t i);
  bool poolGeometry(const Op& op, const Normalised& n, pml_hip_pool2d_desc* d, Spatial* sy, Spatial* sx);
  bool tryGlobalPool(size_t i);
  bool tryPool(size_t i);
  bool isWindowIota(const ValuePtr& ix, int64_t kh, int64_t kw);
  bool matchWindowArgmax(size_t ui, const Op& pool, const pml_hip_pool2d_desc& pd);
  static bool reducesLastAxis(const Op& op, AggKind agg);
  bool trySoftmax(size_t i);

  // ----- the general contraction kernel ---------------------------------------------------

  static std::vector<int> choosePivots(const Op& op);
  void emitGeneral(size_t i);
};

}  // namespace pmlc::target::hip

#include "hip_plan.h"

#include <algorithm>
#include <array>
#include <cstring>
#include <fstream>
#include <map>
#include <numeric>
#include <set>
#include <sstream>

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

namespace {

int hipType(DataType dt) { return static_cast<int>(dt); }  // the kernel library uses plaidml_datatype values

int hipAgg(AggKind a) {
  switch (a) {
    case AggKind::assign: return PML_HIP_AGG_ASSIGN;
    case AggKind::add: return PML_HIP_AGG_ADD;
    case AggKind::max: return PML_HIP_AGG_MAX;
    case AggKind::min: return PML_HIP_AGG_MIN;
    case AggKind::mul: return PML_HIP_AGG_MUL;
  }
  return 0;
}
int hipCombo(ComboKind c) {
  switch (c) {
    case ComboKind::none: return PML_HIP_COMBO_NONE;
    case ComboKind::add: return PML_HIP_COMBO_ADD;
    case ComboKind::cond: return PML_HIP_COMBO_COND;
    case ComboKind::eq: return PML_HIP_COMBO_EQ;
    case ComboKind::mul: return PML_HIP_COMBO_MUL;
  }
  return 0;
}

bool is64(DataType dt) { return util::byteSize(dt) == 8; }

// A contraction with its range-1 indices folded into the constants.
struct Normalised {
  size_t nIdx = 0;
  std::vector<bool> active;
  std::vector<std::vector<Affine>> acc;  // [0] sink, [1..] sources
  std::vector<tile::ConstraintForm> cons;
};

Normalised normalise(const Op& op) {
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
void formRange(const Op& op, const Affine& a, int64_t* lo, int64_t* hi) {
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
bool impliedByBox(const Op& op, const Affine& a, int64_t size) {
  if (a.den != 1) return false;
  int64_t lo, hi;
  formRange(op, a, &lo, &hi);
  return lo >= 0 && hi < size;
}

bool emptyBox(const Op& op) {
  for (size_t v = 0; v < op.lower.size(); ++v)
    if (op.lower[v] > op.upper[v]) return true;
  return false;
}

// flat element stride of every index in one access (plain multiples only); false if a form has den != 1
bool indexStrides(const std::vector<Affine>& forms, const TensorShape& shape, std::vector<int64_t>* strides,
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

  std::shared_ptr<Plan> run() {
    rewriteSelectMinMax();
    tile::eliminateDeadOps(prog_);
    analyse();
    for (size_t i = 0; i < prog_->inputs.size(); ++i) {
      BufferInfo b;
      b.kind = BufferInfo::Input;
      b.index = static_cast<int>(i);
      b.bytes = prog_->inputs[i]->shape.getByteSize();
      b.name = prog_->inputs[i]->name;
      plan_->buffers.push_back(b);
      bufferOf_[prog_->inputs[i].get()] = static_cast<int>(plan_->buffers.size()) - 1;
      plan_->input_buffers.push_back(static_cast<int>(plan_->buffers.size()) - 1);
    }
    // outputs: the first occurrence of a Temp value owns an Output buffer; anything else is copied
    plan_->output_buffers.assign(prog_->outputs.size(), -1);
    std::vector<std::pair<size_t, ValuePtr>> copies;
    for (size_t i = 0; i < prog_->outputs.size(); ++i) {
      const ValuePtr& v = prog_->outputs[i];
      BufferInfo b;
      b.kind = BufferInfo::Output;
      b.index = static_cast<int>(i);
      b.bytes = v->shape.getByteSize();
      b.name = v->name;
      plan_->buffers.push_back(b);
      const int id = static_cast<int>(plan_->buffers.size()) - 1;
      plan_->output_buffers[i] = id;
      if (v->kind == Value::Temp && !bufferOf_.count(v.get()))
        bufferOf_[v.get()] = id;
      else
        copies.emplace_back(i, v);
    }
    for (size_t i = 0; i < prog_->ops.size(); ++i) {
      if (consumed_.count(i)) continue;
      emit(i);
    }
    for (const auto& c : copies) {
      Step s;
      s.kind = Step::Copy;
      s.a = bufferFor(c.second);
      s.c = plan_->output_buffers[c.first];
      s.copy_bytes = c.second->shape.getByteSize();
      s.text = "copy -> output #" + std::to_string(c.first);
      plan_->steps.push_back(s);
    }
    if (opt_.fuse && opt_.specialise) fuseSecondProducts();
    if (opt_.specialise) padDepthwiseResults();
    pruneDeadSteps();
    applySchedule();
    return plan_;
  }

  // Tiling overrides, per program (target options) and per step (schedule file): they travel to the kernel library in
  // the descriptors' schedule bits.  Runs last, so that a step is keyed by the text the plan dump shows for it.
  static int convPathByName(const std::string& name) {
    static const char* const names[] = {"auto", "igemm", "patches", "ldsfilter", "blocks"};
    for (int i = 0; i < 5; ++i)
      if (name == names[i]) return i;
    throw std::runtime_error("Invalid convolution path '" + name + "' (igemm, patches, ldsfilter or blocks)");
  }
  static int tileByName(const std::string& name) {
    const int t = pml_hip_tile_by_name(name.c_str());
    if (t < 0) throw std::runtime_error("Invalid tile '" + name + "' (64x64, 128x64, 128x128, 128x64w8, 128x128w8, 128x128w8s2, 256x128w16, 64x64w8k2, 256x256w8, 128x64n2, 192x384w8, 64x64ks)");
    return t;
  }
  struct Rule {
    int tile = -1, conv = 0;
  };
  static Rule parseRule(const std::string& text) {  // "tile=...,conv=..."
    Rule r;
    std::stringstream ss(text);
    for (std::string item; std::getline(ss, item, ',');) {
      const auto eq = item.find('=');
      const std::string key = item.substr(0, eq), value = eq == std::string::npos ? "" : item.substr(eq + 1);
      if (key == "tile")
        r.tile = tileByName(value);
      else if (key == "conv")
        r.conv = convPathByName(value);
      else
        throw std::runtime_error("Invalid schedule entry '" + item + "' (tile=... or conv=...)");
    }
    return r;
  }
  void applySchedule() {
    Rule all;
    if (!opt_.tile.empty()) all.tile = tileByName(opt_.tile);
    if (!opt_.conv.empty()) all.conv = convPathByName(opt_.conv);
    std::map<std::string, Rule> rules;
    if (!opt_.schedule_path.empty()) {
      std::ifstream f(opt_.schedule_path);
      if (!f) throw std::runtime_error("Cannot read the schedule file " + opt_.schedule_path);
      for (std::string line; std::getline(f, line);) {
        const auto open = line.rfind(" {"), lead = line.find("] ");
        if (line.empty() || line.back() != '}' || open == std::string::npos || lead == std::string::npos || lead > open) continue;
        rules[line.substr(lead + 2, open - lead - 2)] = parseRule(line.substr(open + 2, line.size() - open - 3));
      }
    }
    for (Step& s : plan_->steps) {
      if (s.kind != Step::Gemm && s.kind != Step::Conv2d) continue;
      Rule r = all;
      const auto it = rules.find(s.text);
      if (it != rules.end()) {
        if (it->second.tile >= 0) r.tile = it->second.tile;
        if (it->second.conv > 0) r.conv = it->second.conv;
      }
      if (s.kind == Step::Gemm) r.conv = 0;
      int32_t& flags = s.kind == Step::Gemm ? s.gemm.flags : s.conv.flags;
      std::string text;
      if (r.tile >= 0) {
        flags |= PML_HIP_FLAG_TILE(r.tile);
        text += std::string("tile=") + pml_hip_tile_name(r.tile);
      }
      if (r.conv > 0) {
        static const char* const names[] = {"auto", "igemm", "patches", "ldsfilter", "blocks"};
        flags |= PML_HIP_FLAG_CONV(r.conv);
        text += std::string(text.empty() ? "" : ",") + "conv=" + names[r.conv];
      }
      if (!text.empty()) s.schedule = " {" + text + "}";
    }
  }

  // Two matrix products that are added -- a residual block's projection shortcut and the last 1x1 convolution
  // of its main path -- become one launch that accumulates both into the same result tile: the sum is never
  // written and read back (the reference reaches the same by fusing the loop nests of producer and consumer,
  // pmlc/target/x86/pipeline.cc:304-322).  Works on finished steps: Y = gemm / 1x1 convolution whose tail starts
  // with "+ result of X", X = earlier gemm / 1x1 convolution without a tail whose result nobody else reads.
  void fuseSecondProducts() {
    auto pointwise = [](const Step& s) {
      const pml_hip_conv2d_desc& c = s.conv;
      return s.kind == Step::Conv2d && c.kh == 1 && c.kw == 1 && c.pad_h == 0 && c.pad_w == 0 && c.dil_h == 1 && c.dil_w == 1 &&
             c.stride_h == c.stride_w && c.in_dtype == PML_HIP_BF16 && c.out_dtype == PML_HIP_BF16;
    };
    auto plainGemm = [](const Step& s) {
      return s.kind == Step::Gemm && s.gemm.k2 == 0 && s.gemm.in_dtype == PML_HIP_BF16 && s.gemm.out_dtype == PML_HIP_BF16 &&
             s.gemm.ldc == s.gemm.n && s.c_off == 0;
    };
    auto columnInit = [](int32_t kind, int32_t dtype, int64_t rs, int64_t cs) {
      return kind == 0 || (kind == 1 && dtype == PML_HIP_BF16 && rs == 0 && cs == 1);
    };
    for (size_t y = 0; y < plan_->steps.size(); ++y) {
      Step& Y = plan_->steps[y];
      if (!plainGemm(Y) && !pointwise(Y)) continue;
      const pml_hip_epilogue& ty = Y.kind == Step::Gemm ? Y.gemm.tail : Y.conv.tail;
      if (ty.n_ops < 1 || ty.ops[0].opcode != PML_HIP_EPI_ADD || ty.ops[0].operand_kind != PML_HIP_OPND_TENSOR ||
          ty.ops[0].dtype != PML_HIP_BF16)
        continue;
      const int q = ty.ops[0].operand;
      const int64_t n_cols = Y.kind == Step::Gemm ? Y.gemm.n : Y.conv.co;
      if (q < 0 || q >= ty.n_operands || ty.operand_dtype[q] != PML_HIP_BF16 || ty.operand_col_stride[q] != 1 ||
          ty.operand_row_stride[q] != n_cols || static_cast<size_t>(q) >= Y.operands.size() || Y.operand_off[q] != 0)
        continue;
      bool reused = false;  // the operand must not be used again further down the tail
      for (int k = 1; k < ty.n_ops; ++k) reused = reused || (ty.ops[k].operand_kind == PML_HIP_OPND_TENSOR && ty.ops[k].operand == q);
      if (reused) continue;
      const int xbuf = Y.operands[q];
      if (plan_->buffers[xbuf].kind != BufferInfo::Temp) continue;
      // X: the last earlier writer of that buffer; readers: only Y's tail
      int x = -1;
      for (size_t k = 0; k < y; ++k)
        if (plan_->steps[k].c == xbuf) x = static_cast<int>(k);
      if (x < 0) continue;
      int readers = 0;
      for (const Step& s : plan_->steps) {
        for (int r : {s.a, s.b, s.init, s.a2, s.b2, s.init2}) readers += r == xbuf;
        for (int r : s.operands) readers += r == xbuf;
      }
      if (readers != 1) continue;
      const Step& X = plan_->steps[x];
      if (!plainGemm(X) && !pointwise(X)) continue;
      const pml_hip_epilogue& tx = X.kind == Step::Gemm ? X.gemm.tail : X.conv.tail;
      if (tx.n_ops != 0 || !X.outs.empty()) continue;
      // one of the two must be a plain GEMM (the kernel's first product walks plain rows)
      const Step& P = plainGemm(Y) ? Y : X;   // first product
      const Step& S = plainGemm(Y) ? X : Y;   // second product
      if (!plainGemm(P) || &P == &S) continue;
      if (P.gemm.b_layout != 0 || P.b_is_nk) continue;
      const pml_hip_gemm_desc& pg = P.gemm;
      Step F = P;
      pml_hip_gemm_desc& g = F.gemm;
      if (S.kind == Step::Gemm) {
        const pml_hip_gemm_desc& sg = S.gemm;
        if (sg.m != pg.m || sg.n != pg.n || sg.b_layout != 0 || S.b_is_nk) continue;
        if (!columnInit(sg.init_kind, sg.init_dtype, sg.init_row_stride, sg.init_col_stride) || S.init_off != 0) continue;
        g.k2 = sg.k;
        g.lda2 = sg.lda;
        g.ldb2 = sg.ldb;
        g.a2_stride = 0;
        g.init2_kind = sg.init_kind;
      } else {
        const pml_hip_conv2d_desc& sc = S.conv;
        if (sc.n * sc.oh * sc.ow != pg.m || sc.co != pg.n) continue;
        if (!columnInit(sc.init_kind, sc.init_dtype, sc.init_row_stride, sc.init_col_stride) || S.init_off != 0) continue;
        g.k2 = sc.ci;
        g.lda2 = sc.ci;
        g.ldb2 = sc.co;
        const bool plain_rows = sc.stride_h == 1 && sc.oh == sc.h && sc.ow == sc.w;
        g.a2_stride = plain_rows ? 0 : static_cast<int32_t>(sc.stride_h);
        g.a2_h = sc.h;
        g.a2_w = sc.w;
        g.a2_oh = sc.oh;
        g.a2_ow = sc.ow;
        g.init2_kind = sc.init_kind;
      }
      if ((g.k2 * 2) % 16 != 0 || (g.lda2 * 2) % 16 != 0) continue;
      if (!columnInit(pg.init_kind, pg.init_dtype, pg.init_row_stride, pg.init_col_stride)) continue;
      // the tail is Y's without its first step; operand q goes, later operands move down
      pml_hip_epilogue t{};
      t.n_ops = ty.n_ops - 1;
      for (int k = 1; k < ty.n_ops; ++k) {
        t.ops[k - 1] = ty.ops[k];
        if (t.ops[k - 1].operand_kind == PML_HIP_OPND_TENSOR && t.ops[k - 1].operand > q) t.ops[k - 1].operand -= 1;
      }
      t.n_operands = ty.n_operands - 1;
      for (int k = 0, w = 0; k < ty.n_operands; ++k) {
        if (k == q) continue;
        t.operand_dtype[w] = ty.operand_dtype[k];
        t.operand_row_stride[w] = ty.operand_row_stride[k];
        t.operand_col_stride[w] = ty.operand_col_stride[k];
        ++w;
      }
      g.tail = t;
      g.c_dtype = Y.kind == Step::Gemm ? Y.gemm.c_dtype : Y.conv.c_dtype;
      F.c = Y.c;
      F.c_off = 0;
      F.operands.clear();
      F.operand_off.clear();
      for (size_t k = 0; k < Y.operands.size(); ++k) {
        if (static_cast<int>(k) == q) continue;
        F.operands.push_back(Y.operands[k]);
        F.operand_off.push_back(k < Y.operand_off.size() ? Y.operand_off[k] : 0);
      }
      F.outs = Y.outs;
      F.out2 = Y.out2;
      F.a2 = S.a;
      F.b2 = S.b;
      F.init2 = S.init;
      F.a2_off = S.a_off;
      F.b2_off = S.b_off;
      F.b2_constant = S.b_constant;
      F.flops = X.flops + Y.flops;
      F.bytes = X.bytes + Y.bytes - 2.0 * static_cast<double>(pg.m * pg.n) * 2;  // the sum is neither written nor read
      {
        TailBuild shown;
        shown.tail = t;
        std::stringstream ss;
        ss << "gemm bf16 m=" << g.m << " n=" << g.n << " k=" << g.k << " + second product k2=" << g.k2;
        if (S.kind == Step::Conv2d) ss << " (pixel rows of a 1x1 convolution, stride " << S.conv.stride_h << ")";
        ss << " B=[k][n]" << ((F.b_constant && F.b2_constant) ? " (constants, packed once)" : "") << (g.init_kind ? " +init" : "")
           << (g.init2_kind ? " +init2" : "") << tailText(shown);
        const std::string& ytext = Y.text;
        const size_t arrow = ytext.rfind(" -> ");
        ss << (arrow == std::string::npos ? "" : ytext.substr(arrow));
        F.text = ss.str();
      }
      plan_->steps[y] = F;  // X is left without readers and is dropped by pruneDeadSteps
    }
  }

  // A depthwise convolution whose result is a temporary that only one matrix product reads as its left-hand rows
  // (the depthwise-separable block): when a pixel's channels do not fill whole 128-byte lines (728 bf16 = 1456
  // bytes), the temporary gets a row pitch that does, so every GEMM row starts on a line; the depthwise kernel
  // writes with that pitch, the GEMM reads with it as its leading dimension.  The layout of a temporary is the
  // planner's to choose (the reference sizes and places its temporaries itself too, pmlc/target/x86/pipeline.cc:289-360).
  void padDepthwiseResults() {
    for (size_t x = 0; x < plan_->steps.size(); ++x) {
      Step& X = plan_->steps[x];
      if (X.kind != Step::Dwconv2d || X.dw.tail.n_ops != 0 || !X.outs.empty() || X.c < 0) continue;
      if (plan_->buffers[X.c].kind != BufferInfo::Temp) continue;
      const int es = X.dw.dtype == PML_HIP_F32 ? 4 : 2;
      const int64_t row_bytes = X.dw.c * es;
      if (row_bytes % 128 == 0 || row_bytes < 512) continue;
      const int64_t pitch = (row_bytes + 127) / 128 * 128 / es;
      const int64_t rows = X.dw.n * X.dw.oh * X.dw.ow;
      // (the matrix-core kernels address their left-hand side with 32-bit byte offsets below 2 GiB)
      if (pitch >= (int64_t{1} << 31) || rows * pitch * es >= (int64_t{1} << 31)) continue;
      int readers = 0, writers = 0, y = -1;
      for (size_t k = 0; k < plan_->steps.size(); ++k) {
        const Step& s = plan_->steps[k];
        for (int r : {s.a, s.b, s.init, s.a2, s.b2, s.init2}) readers += r == X.c;
        for (int r : s.operands) readers += r == X.c;
        writers += s.c == X.c;
        writers += s.out2 == X.c;
        for (int w : s.outs) writers += w == X.c;
        if (s.a == X.c && k > x) y = static_cast<int>(k);
      }
      if (readers != 1 || writers != 1 || y < 0) continue;
      Step& Y = plan_->steps[y];
      if (Y.kind != Step::Gemm || Y.a_off != 0 || Y.gemm.m != rows || Y.gemm.k != X.dw.c || Y.gemm.lda != X.dw.c) continue;
      X.dw.out_pitch = static_cast<int32_t>(pitch);
      Y.gemm.lda = pitch;
      plan_->buffers[X.c].bytes = static_cast<size_t>(rows * pitch * es);
      X.text += " (row pitch " + std::to_string(pitch) + ")";
      Y.text += " (lda " + std::to_string(pitch) + ")";
    }
  }

  // A kernel that took over the work of earlier operations (the int8 GEMM reads the un-cast operands, a pool
  // kernel also writes the window argmax) can leave launches whose results nobody reads: drop them.
  void pruneDeadSteps() {
    std::set<int> needed;
    for (int b : plan_->output_buffers) needed.insert(b);
    std::vector<Step> kept;
    for (auto it = plan_->steps.rbegin(); it != plan_->steps.rend(); ++it) {
      const Step& s = *it;
      std::vector<int> writes = {s.c, s.out2};
      writes.insert(writes.end(), s.outs.begin(), s.outs.end());
      bool live = false;
      for (int w : writes) live = live || (w >= 0 && needed.count(w));
      if (!live) continue;
      // a full overwrite ends the need for earlier writers of the same buffer, except for the general
      // contraction, which accumulates into a pre-filled output
      const bool accumulates = s.kind == Step::Contract && s.con.has_init;
      if (!accumulates)
        for (int w : writes) needed.erase(w);
      for (int r : {s.a, s.b, s.init, s.a2, s.b2, s.init2}) {
        if (r >= 0) needed.insert(r);
      }
      for (int r : s.operands) needed.insert(r);
      if (accumulates) needed.insert(s.c);
      kept.push_back(s);
    }
    std::reverse(kept.begin(), kept.end());
    plan_->steps = kept;
  }

 private:
  Program* prog_;
  Options opt_;
  std::shared_ptr<Plan> plan_;
  std::map<const Value*, int> bufferOf_;
  std::map<const Value*, std::vector<size_t>> users_;
  std::map<const Value*, size_t> producer_;
  std::set<const Value*> outputs_;
  std::set<size_t> consumed_;

  void analyse() {
    users_.clear();
    producer_.clear();
    outputs_.clear();
    for (size_t i = 0; i < prog_->ops.size(); ++i) {
      const Op& op = prog_->ops[i];
      producer_[op.result.get()] = i;
      for (const ValuePtr& v : op.operands) users_[v.get()].push_back(i);
      if (op.init) users_[op.init.get()].push_back(i);
    }
    for (const ValuePtr& v : prog_->outputs) outputs_.insert(v.get());
  }

  // select(cmp_lt(a, b), b, a) -> max(a, b);  select(cmp_lt(a, b), a, b) -> min(a, b)
  void rewriteSelectMinMax() {
    std::map<const Value*, size_t> producer;
    std::map<const Value*, int> uses;
    for (size_t i = 0; i < prog_->ops.size(); ++i) {
      producer[prog_->ops[i].result.get()] = i;
      for (const ValuePtr& v : prog_->ops[i].operands) uses[v.get()]++;
    }
    for (const ValuePtr& v : prog_->outputs) uses[v.get()]++;
    for (Op& op : prog_->ops) {
      if (op.kind != Op::Eltwise || op.fn != "select" || op.operands.size() != 3) continue;
      auto it = producer.find(op.operands[0].get());
      if (it == producer.end()) continue;
      const Op& cmp = prog_->ops[it->second];
      if (cmp.kind != Op::Eltwise || (cmp.fn != "cmp_lt" && cmp.fn != "cmp_gt") || cmp.operands.size() != 2) continue;
      const ValuePtr &a = cmp.operands[0], &b = cmp.operands[1];
      // the running value of a chain has to be the first comparand
      if (a->kind == Value::Literal) continue;
      const ValuePtr &t = op.operands[1], &f = op.operands[2];
      auto same = [](const ValuePtr& x, const ValuePtr& y) {
        if (x == y) return true;
        // two scalar literals / rank-0 constants with the same value count as the same operand
        // (an untyped literal takes the type of the tensor it meets, so `x > -127.0` and `cast(-127.0, f32)` agree)
        if (x->kind == Value::Literal && y->kind == Value::Literal) {
          const DataType xt = x->shape.elementType, yt = y->shape.elementType;
          if (xt != yt && !util::isAmbiguous(xt) && !util::isAmbiguous(yt)) return false;
          return x->literalAsDouble() == y->literalAsDouble();
        }
        return false;
      };
      // the comparison happens in the promoted type of (a, b); min/max in the chain must compute the same
      if (a->shape.elementType != b->shape.elementType && a->kind != Value::Literal && b->kind != Value::Literal) continue;
      if (cmp.fn == "cmp_gt") {
        // select(a > b, a, b): the lower bound of op::clip
        if (same(t, a) && same(f, b)) {
          op.fn = "maxgt";
          op.operands = {a, b};
        }
      } else if (same(t, b) && same(f, a)) {
        op.fn = "max";
        op.operands = {a, b};
      } else if (same(t, a) && same(f, b)) {
        op.fn = "min";
        op.operands = {a, b};
      }
    }
  }

  int newBuffer(BufferInfo::Kind kind, size_t bytes, const std::string& name) {
    BufferInfo b;
    b.kind = kind;
    b.bytes = bytes;
    b.name = name;
    plan_->buffers.push_back(b);
    return static_cast<int>(plan_->buffers.size()) - 1;
  }

  int bufferFor(const ValuePtr& v) {
    auto it = bufferOf_.find(v.get());
    if (it != bufferOf_.end()) return it->second;
    int id = -1;
    switch (v->kind) {
      case Value::Constant:
        id = newBuffer(BufferInfo::Constant, v->constant->size(), v->name);
        plan_->buffers[id].constant = v->constant;
        break;
      case Value::Temp:
        id = newBuffer(BufferInfo::Temp, v->shape.getByteSize(), v->name);
        break;
      case Value::Literal:
        throw std::runtime_error("internal: a scalar literal has no buffer");
      case Value::Input:
        throw std::runtime_error("internal: unknown program input");
    }
    bufferOf_[v.get()] = id;
    return id;
  }

  // a one-element constant of type dt holding the given value
  int scalarConstant(DataType dt, double f, int64_t i) {
    TensorShape shape(dt);
    auto buf = std::make_shared<util::SimpleBuffer>(shape);
    char* p = buf->data();
    switch (dt) {
      case DataType::f32: { float x = static_cast<float>(f); std::memcpy(p, &x, 4); break; }
      case DataType::f64: std::memcpy(p, &f, 8); break;
      case DataType::bf16: {
        float x = static_cast<float>(f);
        uint32_t u;
        std::memcpy(&u, &x, 4);
        uint16_t h = (u & 0x7fffffffu) > 0x7f800000u ? static_cast<uint16_t>((u >> 16) | 0x40)
                                                     : static_cast<uint16_t>((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
        std::memcpy(p, &h, 2);
        break;
      }
      case DataType::f16: throw std::runtime_error("float16 constants are not supported by the hip target");
      default: std::memcpy(p, &i, util::byteSize(dt)); break;
    }
    const int id = newBuffer(BufferInfo::Constant, buf->size(), "scalar");
    plan_->buffers[id].constant = buf;
    return id;
  }

  // ----- elementwise chains -------------------------------------------------------------

  static int unaryOpcode(const std::string& fn) {
    static const std::map<std::string, int> m = {
        {"relu", PML_HIP_EPI_RELU}, {"neg", PML_HIP_EPI_NEG},     {"exp", PML_HIP_EPI_EXP},   {"log", PML_HIP_EPI_LOG},
        {"sqrt", PML_HIP_EPI_SQRT}, {"tanh", PML_HIP_EPI_TANH},   {"floor", PML_HIP_EPI_FLOOR}, {"ceil", PML_HIP_EPI_CEIL},
        {"round", PML_HIP_EPI_ROUND}, {"sin", PML_HIP_EPI_SIN},     {"cos", PML_HIP_EPI_COS},   {"tan", PML_HIP_EPI_TAN},
        {"sinh", PML_HIP_EPI_SINH}, {"cosh", PML_HIP_EPI_COSH},   {"asin", PML_HIP_EPI_ASIN}, {"acos", PML_HIP_EPI_ACOS},
        {"atan", PML_HIP_EPI_ATAN}, {"asinh", PML_HIP_EPI_ASINH}, {"acosh", PML_HIP_EPI_ACOSH}, {"atanh", PML_HIP_EPI_ATANH},
        {"erf", PML_HIP_EPI_ERF},   {"bit_not", PML_HIP_EPI_BIT_NOT}, {"logical_not", PML_HIP_EPI_LOGICAL_NOT}};
    auto it = m.find(fn);
    return it == m.end() ? 0 : it->second;
  }
  // The operand types an operation accepts (the OperandsAre / ResultIs predicates of the eltwise pattern
  // table, pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:1271-1385): `dt` is the type the step computes in.
  static void checkStepType(const std::string& fn, DataType dt) {
    static const std::set<std::string> float_only = {"sin",  "cos",   "tan",   "sinh",  "cosh", "asin", "acos",
                                                     "atan", "asinh", "acosh", "atanh", "erf",  "pow"};
    static const std::set<std::string> int_only = {"bit_and", "bit_or", "bit_xor", "bit_not", "bit_shl", "bit_shr"};
    if (float_only.count(fn) && !util::isFloat(dt))
      throw std::runtime_error("'" + fn + "' needs floating-point operands, got " + util::mnemonic(dt));
    if (int_only.count(fn) && !util::isInteger(dt))
      throw std::runtime_error("'" + fn + "' needs integer operands, got " + util::mnemonic(dt));
  }
  // comparisons and truth-value operations compute in their operands' promoted type and yield i1
  static bool computesInOperandType(const std::string& fn) { return ast::isCompareOp(fn) || ast::isLogicalOp(fn); }
  // opcode when the running value is the first / second operand (0 = not expressible)
  static int binaryOpcode(const std::string& fn, bool running_first) {
    struct E { int first, second; };
    static const std::map<std::string, E> m = {
        {"add", {PML_HIP_EPI_ADD, PML_HIP_EPI_ADD}},       {"sub", {PML_HIP_EPI_SUB, PML_HIP_EPI_RSUB}},
        {"mul", {PML_HIP_EPI_MUL, PML_HIP_EPI_MUL}},       {"div", {PML_HIP_EPI_DIV, PML_HIP_EPI_RDIV}},
        {"max", {PML_HIP_EPI_MAX, 0}},                     {"min", {PML_HIP_EPI_MIN, 0}},
        {"maxgt", {PML_HIP_EPI_MAX_GT, 0}},
        {"pow", {PML_HIP_EPI_POW, PML_HIP_EPI_RPOW}},      {"mod", {PML_HIP_EPI_MOD, PML_HIP_EPI_RMOD}},
        {"bit_and", {PML_HIP_EPI_BIT_AND, PML_HIP_EPI_BIT_AND}}, {"bit_or", {PML_HIP_EPI_BIT_OR, PML_HIP_EPI_BIT_OR}},
        {"bit_xor", {PML_HIP_EPI_BIT_XOR, PML_HIP_EPI_BIT_XOR}}, {"bit_shl", {PML_HIP_EPI_SHL, PML_HIP_EPI_RSHL}},
        {"bit_shr", {PML_HIP_EPI_SHR, PML_HIP_EPI_RSHR}},
        {"logical_and", {PML_HIP_EPI_LOGICAL_AND, PML_HIP_EPI_LOGICAL_AND}},
        {"logical_or", {PML_HIP_EPI_LOGICAL_OR, PML_HIP_EPI_LOGICAL_OR}},
        {"logical_xor", {PML_HIP_EPI_LOGICAL_XOR, PML_HIP_EPI_LOGICAL_XOR}},
        {"cmp_lt", {PML_HIP_EPI_CMP_LT, PML_HIP_EPI_CMP_GT}}, {"cmp_gt", {PML_HIP_EPI_CMP_GT, PML_HIP_EPI_CMP_LT}},
        {"cmp_le", {PML_HIP_EPI_CMP_LE, PML_HIP_EPI_CMP_GE}}, {"cmp_ge", {PML_HIP_EPI_CMP_GE, PML_HIP_EPI_CMP_LE}},
        {"cmp_eq", {PML_HIP_EPI_CMP_EQ, PML_HIP_EPI_CMP_EQ}}, {"cmp_ne", {PML_HIP_EPI_CMP_NE, PML_HIP_EPI_CMP_NE}}};
    auto it = m.find(fn);
    if (it == m.end()) return 0;
    return running_first ? it->second.first : it->second.second;
  }

  // Broadcast strides of `shape` against the output shape `out` (trailing alignment).
  static bool ndStrides(const TensorShape& shape, const TensorShape& out, std::array<int64_t, PML_HIP_MAX_RANK>* st) {
    st->fill(0);
    const size_t ro = out.getRank(), rs = shape.getRank();
    if (rs > ro || ro > PML_HIP_MAX_RANK) return false;
    const auto dense = shape.denseStrides();
    for (size_t i = 0; i < rs; ++i) {
      const size_t od = ro - rs + i;
      if (shape.sizes[i] == out.sizes[od])
        (*st)[od] = shape.sizes[i] == 1 ? 0 : dense[i];
      else if (shape.sizes[i] == 1)
        (*st)[od] = 0;
      else
        return false;
    }
    return true;
  }

  // (row, col) strides of an operand against an output seen as rows x cols (cols = last dimension)
  static bool rowColStrides(const TensorShape& shape, const TensorShape& out, int64_t* rs, int64_t* cs) {
    if (out.getRank() == 0) return false;
    const int64_t cols = out.sizes.back();
    if (shape.elements() == 1) {
      *rs = 0;
      *cs = 0;
      return true;
    }
    if (shape.sizes == out.sizes) {
      *rs = cols;
      *cs = 1;
      return true;
    }
    if (shape.getRank() > out.getRank()) return false;
    // vector along the last dimension
    bool vec = shape.sizes.back() == cols;
    for (size_t i = 0; i + 1 < shape.getRank(); ++i) vec = vec && shape.sizes[i] == 1;
    if (vec) {
      *rs = 0;
      *cs = 1;
      return true;
    }
    // one value per row
    if (shape.getRank() == out.getRank() && shape.sizes.back() == 1) {
      bool lead = true;
      for (size_t i = 0; i + 1 < shape.getRank(); ++i) lead = lead && shape.sizes[i] == out.sizes[i];
      if (lead) {
        *rs = 1;
        *cs = 0;
        return true;
      }
    }
    return false;
  }

  // Extends a chain from `value` (produced by op `root` or being the loaded input).  `two_d`
  // selects the (row, col) operand addressing of the dense kernels; otherwise N-d strides are
  // recorded.  `allow64` is false for the kernels whose tail interpreter is 32-bit.
  void extendTail(TailBuild* tb, ValuePtr value, size_t root, bool two_d, bool allow64) {
    tb->final_value = value;
    tb->final_dtype = value->shape.elementType;
    if (!opt_.fuse) return;
    for (;;) {
      const ValuePtr cur = tb->final_value;
      const auto uit = users_.find(cur.get());
      if (uit == users_.end()) return;
      // candidate: the first not-yet-consumed user; every other use keeps the value alive via STORE
      std::vector<size_t> users;
      for (size_t u : uit->second)
        if (!consumed_.count(u)) users.push_back(u);
      std::sort(users.begin(), users.end());
      users.erase(std::unique(users.begin(), users.end()), users.end());
      if (users.empty()) return;
      const bool extra_uses = users.size() > 1 || outputs_.count(cur.get());
      const size_t ui = users.front();
      const Op& u = prog_->ops[ui];
      if (u.kind != Op::Eltwise && u.kind != Op::Cast) return;
      if (u.result->shape.sizes != cur->shape.sizes) return;
      if (tb->tail.n_ops + 2 > PML_HIP_MAX_EPI_OPS) return;
      const DataType rdt = u.result->shape.elementType;
      pml_hip_epi_op step{};
      int add_operand_buf = -1;
      int64_t rs = 0, cs = 0;
      std::array<int64_t, PML_HIP_MAX_RANK> nd{};
      DataType operand_dt = DataType::invalid;
      if (u.kind == Op::Cast) {
        if (!allow64 && (is64(rdt) || is64(cur->shape.elementType))) return;
        step.opcode = PML_HIP_EPI_CAST;
        step.dtype = hipType(rdt);
      } else if (u.operands.size() == 1) {
        if (u.fn == "ident") {
          step.opcode = 0;  // no step, the value passes through
        } else {
          step.opcode = unaryOpcode(u.fn);
          if (!step.opcode) return;
          const DataType sdt = computesInOperandType(u.fn) ? cur->shape.elementType : rdt;
          checkStepType(u.fn, sdt);
          step.dtype = hipType(sdt);
          if (!allow64 && is64(sdt)) return;
        }
        if (!allow64 && is64(rdt)) return;
      } else if (u.operands.size() == 2) {
        const bool first = u.operands[0] == cur;
        if ((u.operands[0] == cur) == (u.operands[1] == cur)) return;  // x op x, or not an operand
        const ValuePtr& other = first ? u.operands[1] : u.operands[0];
        step.opcode = binaryOpcode(u.fn, first);
        if (!step.opcode) return;
        // arithmetic happens in the promoted operand type; comparisons too, their result is i1
        DataType cdt = rdt;
        if (computesInOperandType(u.fn)) {
          cdt = other->kind == Value::Literal ? cur->shape.elementType
                                              : util::promoteTypes(cur->shape.elementType, other->shape.elementType);
        }
        checkStepType(u.fn, cdt);
        if (!allow64 && (is64(cdt) || is64(other->shape.elementType))) return;
        step.dtype = hipType(cdt);
        if (other->kind == Value::Literal) {
          step.operand_kind = PML_HIP_OPND_IMM;
          step.imm = other->literalAsDouble();
        } else {
          // must already exist when the fused kernel runs
          if (other->kind == Value::Temp) {
            auto pit = producer_.find(other.get());
            if (pit == producer_.end() || pit->second >= root || !bufferOf_.count(other.get())) return;
          }
          if (tb->tail.n_operands >= PML_HIP_MAX_EPI_OPERANDS) return;
          if (two_d) {
            if (!rowColStrides(other->shape, cur->shape, &rs, &cs)) return;
          } else {
            if (!ndStrides(other->shape, cur->shape, &nd)) return;
          }
          step.operand_kind = PML_HIP_OPND_TENSOR;
          add_operand_buf = bufferFor(other);
          operand_dt = other->shape.elementType;
        }
      } else {
        return;
      }
      // commit: keep `cur` alive if something else needs it
      if (extra_uses) {
        if (tb->tail.n_ops + 3 > PML_HIP_MAX_EPI_OPS) return;
        if (static_cast<int>(tb->outs.size()) >= PML_HIP_MAX_EPI_OPERANDS) return;
        pml_hip_epi_op st{};
        st.opcode = PML_HIP_EPI_STORE;
        st.dtype = hipType(cur->shape.elementType);
        st.operand = static_cast<int>(tb->outs.size());
        tb->outs.push_back(bufferFor(cur));
        tb->tail.ops[tb->tail.n_ops++] = st;
      }
      if (add_operand_buf >= 0) {
        const int k = tb->tail.n_operands++;
        step.operand = k;
        tb->tail.operand_dtype[k] = hipType(operand_dt);
        tb->tail.operand_row_stride[k] = rs;
        tb->tail.operand_col_stride[k] = cs;
        tb->operand_bufs.push_back(add_operand_buf);
        tb->operand_offs.push_back(0);
        tb->nd_strides.push_back(nd);
      }
      if (step.opcode) tb->tail.ops[tb->tail.n_ops++] = step;
      consumed_.insert(ui);
      tb->consumed.push_back(ui);
      tb->final_value = u.result;
      tb->final_dtype = rdt;
    }
  }

  static std::string tailText(const TailBuild& tb) {
    if (tb.tail.n_ops == 0) return "";
    static const char* names[] = {"?",    "add",  "sub",   "rsub", "mul",   "div",  "rdiv",  "max",  "min",
                                  "relu", "neg",  "exp",   "log",  "sqrt",  "tanh", "floor", "ceil", "round",
                                  "cast", "store", "lt",   "gt",   "le",    "ge",   "eq",    "ne",   "maxgt",
                                  "sin",  "cos",  "tan",   "sinh", "cosh",  "asin", "acos",  "atan", "asinh",
                                  "acosh", "atanh", "erf", "pow",  "rpow",  "mod",  "rmod",  "and",  "or",
                                  "xor",  "not",  "shl",   "rshl", "shr",   "rshr", "land",  "lor",  "lxor", "lnot"};
    static_assert(sizeof(names) / sizeof(names[0]) == PML_HIP_EPI_LAST_ + 1, "one name per opcode");
    std::stringstream ss;
    ss << " tail=[";
    for (int i = 0; i < tb.tail.n_ops; ++i) {
      const auto& o = tb.tail.ops[i];
      ss << (i ? " " : "") << names[o.opcode];
      if (o.opcode == PML_HIP_EPI_CAST) ss << ":" << util::mnemonic(static_cast<DataType>(o.dtype));
      if (o.operand_kind == PML_HIP_OPND_IMM) ss << "(" << o.imm << ")";
      if (o.operand_kind == PML_HIP_OPND_TENSOR) ss << "(t" << o.operand << ")";
    }
    ss << "]";
    return ss.str();
  }

  void attachTail(Step* s, const TailBuild& tb) {
    s->operands = tb.operand_bufs;
    s->operand_off = tb.operand_offs;
    s->outs = tb.outs;
  }

  // ----- emission -------------------------------------------------------------------------

  void emit(size_t i) {
    const Op& op = prog_->ops[i];
    switch (op.kind) {
      case Op::Contraction: emitContraction(i); break;
      case Op::Eltwise:
      case Op::Cast: emitEltwise(i); break;
      case Op::Index: {
        Step s;
        s.kind = Step::Index;
        s.c = bufferFor(op.result);
        s.index_axis = op.axis;
        s.index_sizes = op.result->shape.sizes;
        s.text = "index axis=" + std::to_string(op.axis) + " -> " + op.result->shape.str();
        plan_->steps.push_back(s);
        break;
      }
      case Op::Special: emitSpecial(i); break;
      case Op::Reshape: {
        Step s;
        s.kind = Step::Copy;
        s.a = bufferFor(op.operands[0]);
        s.c = bufferFor(op.result);
        s.copy_bytes = op.result->shape.getByteSize();
        s.text = "reshape (copy) -> " + op.result->shape.str();
        plan_->steps.push_back(s);
        break;
      }
    }
  }

  // gather / scatter / argsort: one launch each, operands and constants passed through
  void emitSpecial(size_t i) {
    const Op& op = prog_->ops[i];
    auto fill = [](const TensorShape& sh, int64_t* sizes, int32_t* rank, const char* what) {
      if (sh.getRank() > PML_HIP_MAX_SPECIAL_RANK)
        throw std::runtime_error(std::string("'") + what + "' operands of rank > 8 are not supported by the hip target");
      *rank = static_cast<int32_t>(sh.getRank());
      for (size_t d = 0; d < sh.getRank(); ++d) sizes[d] = sh.sizes[d];
    };
    auto param = [&](size_t k) { return static_cast<int64_t>(op.params.at(k)); };
    Step s;
    s.c = bufferFor(op.result);
    for (const ValuePtr& v : op.operands) s.operands.push_back(bufferFor(v));
    if (op.fn == "prng_values" || op.fn == "prng_state") {
      s.kind = Step::Prng;
      s.prng_count = param(0);
      s.prng_state = op.fn == "prng_state";
      s.text = std::string("prng ") + (s.prng_state ? "state after " : "values x ") + std::to_string(s.prng_count) + " -> " +
               op.result->shape.str();
      s.bytes = static_cast<double>(op.result->shape.getByteSize());
    } else if (op.fn == "gather") {
      s.kind = Step::Gather;
      auto& d = s.gat;
      d.dtype = hipType(op.operands[0]->shape.elementType);
      d.idx_dtype = hipType(op.operands[1]->shape.elementType);
      fill(op.operands[0]->shape, d.sizes, &d.rank, "gather");
      fill(op.operands[1]->shape, d.idx_sizes, &d.idx_rank, "gather");
      d.axis = static_cast<int32_t>(param(0));
      d.interpolation = static_cast<int32_t>(param(1));
      d.nearest = static_cast<int32_t>(param(2));
      d.cube_coeff = op.params.at(3);
      d.mode = static_cast<int32_t>(param(4));
      d.batch_dims = static_cast<int32_t>(param(5));
      d.oob = static_cast<int32_t>(param(6));
      if (op.result->shape.getRank() > PML_HIP_MAX_SPECIAL_RANK)
        throw std::runtime_error("'gather' results of rank > 8 are not supported by the hip target");
      if (d.mode == PML_HIP_GATHER_NORMAL && util::isFloat(op.operands[1]->shape.elementType) &&
          util::isFloat(op.operands[0]->shape.elementType) && d.interpolation == PML_HIP_INTERP_NONE)
        throw std::runtime_error("'gather' with floating-point indices needs an interpolation mode");
      s.text = std::string("gather ") + (d.mode == PML_HIP_GATHER_ND ? "nd batch_dims=" + std::to_string(d.batch_dims)
                                                                     : "axis=" + std::to_string(d.axis)) +
               " -> " + op.result->shape.str();
      s.bytes = static_cast<double>(op.result->shape.getByteSize()) * 2 + static_cast<double>(op.operands[1]->shape.getByteSize());
    } else if (op.fn == "scatter") {
      s.kind = Step::Scatter;
      auto& d = s.sca;
      d.dtype = hipType(op.operands[0]->shape.elementType);
      d.idx_dtype = hipType(op.operands[1]->shape.elementType);
      if (op.operands[2]->shape.elementType != op.operands[0]->shape.elementType)
        throw std::runtime_error("'scatter' needs updates of the data's element type, use a cast");
      fill(op.operands[0]->shape, d.sizes, &d.rank, "scatter");
      fill(op.operands[1]->shape, d.idx_sizes, &d.idx_rank, "scatter");
      fill(op.operands[2]->shape, d.upd_sizes, &d.upd_rank, "scatter");
      d.axis = static_cast<int32_t>(param(0));
      d.mode = static_cast<int32_t>(param(1));
      static const char* modes[] = {"normal", "update_slice", "update_elt", "update_nd"};
      s.text = std::string("scatter ") + (d.mode >= 0 && d.mode < 4 ? modes[d.mode] : "?") + " axis=" + std::to_string(d.axis) +
               " -> " + op.result->shape.str();
      s.bytes = static_cast<double>(op.result->shape.getByteSize()) * 2 + static_cast<double>(op.operands[2]->shape.getByteSize()) * 2;
    } else {
      s.kind = Step::ArgSort;
      auto& d = s.srt;
      d.dtype = hipType(op.operands[0]->shape.elementType);
      fill(op.operands[0]->shape, d.sizes, &d.rank, "argsort");
      int64_t axis = param(0);
      if (axis < 0) axis += d.rank;
      if (axis < 0 || axis >= d.rank) throw std::runtime_error("'argsort' axis out of range");
      if (d.sizes[axis] > PML_HIP_MAX_SORT_LINE)
        throw std::runtime_error("'argsort' over more than " + std::to_string(PML_HIP_MAX_SORT_LINE) +
                                 " elements along the axis is not supported by the hip target");
      d.axis = static_cast<int32_t>(axis);
      d.direction = static_cast<int32_t>(param(1));
      s.text = std::string("argsort axis=") + std::to_string(d.axis) + (d.direction ? " desc" : " asc") + " -> " + op.result->shape.str();
      s.bytes = static_cast<double>(op.result->shape.getByteSize()) + static_cast<double>(op.operands[0]->shape.getByteSize());
    }
    plan_->steps.push_back(s);
  }

  void emitEltwise(size_t i) {
    const Op& op = prog_->ops[i];
    const TensorShape& out = op.result->shape;
    if (out.getRank() > PML_HIP_MAX_RANK) throw std::runtime_error("elementwise rank > 6 is not supported by the hip target");
    if (op.kind == Op::Eltwise && op.fn == "select") {
      Step s;
      s.kind = Step::Select;
      s.sel.rank = static_cast<int>(out.getRank());
      std::array<int64_t, PML_HIP_MAX_RANK> st{};
      const ValuePtr* in[3] = {&op.operands[0], &op.operands[1], &op.operands[2]};
      int64_t* dst[3] = {s.sel.cond_strides, s.sel.t_strides, s.sel.f_strides};
      int32_t* dts[3] = {&s.sel.cond_dtype, &s.sel.t_dtype, &s.sel.f_dtype};
      for (int k = 0; k < 3; ++k) {
        ValuePtr v = *in[k];
        if (v->kind == Value::Literal) {
          // a typed scalar (cast of a literal) is read from a one-element constant through zero strides
          if (util::isAmbiguous(v->shape.elementType)) throw std::runtime_error("'select' needs typed operands, use a cast");
          st.fill(0);
          std::copy(st.begin(), st.end(), dst[k]);
          *dts[k] = hipType(v->shape.elementType);
          const bool uns = util::isUnsigned(v->shape.elementType);
          s.operands.push_back(scalarConstant(v->shape.elementType, v->fvalue, uns ? static_cast<int64_t>(v->uvalue) : v->ivalue));
          continue;
        }
        if (!ndStrides(v->shape, out, &st)) throw std::runtime_error("'select' operands do not broadcast");
        std::copy(st.begin(), st.end(), dst[k]);
        *dts[k] = hipType(v->shape.elementType);
        s.operands.push_back(bufferFor(v));
      }
      for (size_t d = 0; d < out.getRank(); ++d) s.sel.sizes[d] = out.sizes[d];
      s.sel.out_dtype = hipType(out.elementType);
      s.c = bufferFor(op.result);
      s.text = "select -> " + out.str();
      s.bytes = static_cast<double>(out.getByteSize()) * 3;
      plan_->steps.push_back(s);
      return;
    }
    // choose the operand that plays the running value: the first tensor operand with the output's shape
    TailBuild tb;
    ValuePtr main;
    int main_pos = -1;
    // max / min keep the first comparand as the running value (their NaN behaviour is not symmetric); it is
    // read through zero strides where it is broadcast
    const bool ordered = op.kind == Op::Eltwise && (op.fn == "max" || op.fn == "min" || op.fn == "maxgt");
    if (ordered && op.operands.size() == 2 && op.operands[0]->kind != Value::Literal) {
      main = op.operands[0];
      main_pos = 0;
    }
    for (size_t k = 0; !main && k < op.operands.size(); ++k) {
      const ValuePtr& v = op.operands[k];
      if (v->kind != Value::Literal && v->shape.sizes == out.sizes) {
        main = v;
        main_pos = static_cast<int>(k);
        break;
      }
    }
    if (!main) {
      // every operand is broadcast: run the chain from the first tensor operand, read through zero strides
      for (size_t k = 0; k < op.operands.size(); ++k) {
        if (op.operands[k]->kind != Value::Literal) {
          main = op.operands[k];
          main_pos = static_cast<int>(k);
          break;
        }
      }
    }
    if (!main) throw std::runtime_error("an elementwise operation over scalar literals only is not supported");
    Step s;
    s.kind = Step::Eltwise;
    s.elt.rank = static_cast<int>(out.getRank());
    for (size_t d = 0; d < out.getRank(); ++d) s.elt.sizes[d] = out.sizes[d];
    std::array<int64_t, PML_HIP_MAX_RANK> st{};
    if (!ndStrides(main->shape, out, &st)) throw std::runtime_error("elementwise operands do not broadcast");
    std::copy(st.begin(), st.end(), s.elt.in_strides);
    s.elt.in_dtype = hipType(main->shape.elementType);
    s.a = bufferFor(main);
    // first step: this op itself, expressed on a pseudo value of the main operand broadcast to `out`
    {
      const DataType rdt = out.elementType;
      pml_hip_epi_op step{};
      if (op.kind == Op::Cast) {
        step.opcode = PML_HIP_EPI_CAST;
        step.dtype = hipType(rdt);
      } else if (op.operands.size() == 1) {
        if (op.fn != "ident") {
          step.opcode = unaryOpcode(op.fn);
          if (!step.opcode) throw std::runtime_error("elementwise operation '" + op.fn + "' is not supported by the hip target");
          const DataType sdt = computesInOperandType(op.fn) ? main->shape.elementType : rdt;
          checkStepType(op.fn, sdt);
          step.dtype = hipType(sdt);
        }
      } else if (op.operands.size() == 2) {
        const bool first = main_pos == 0;
        const ValuePtr& other = op.operands[first ? 1 : 0];
        step.opcode = binaryOpcode(op.fn, first);
        if (!step.opcode && (op.fn == "max" || op.fn == "min")) {
          // running value is the second operand: swap roles by making the other operand the main one is not
          // possible when it is a literal; fall back to an explicit select
          throw std::runtime_error("internal: unsupported operand order for " + op.fn);
        }
        if (!step.opcode) throw std::runtime_error("elementwise operation '" + op.fn + "' is not supported by the hip target");
        DataType cdt = rdt;
        if (computesInOperandType(op.fn))
          cdt = other->kind == Value::Literal ? main->shape.elementType
                                              : util::promoteTypes(main->shape.elementType, other->shape.elementType);
        checkStepType(op.fn, cdt);
        step.dtype = hipType(cdt);
        if (other->kind == Value::Literal) {
          step.operand_kind = PML_HIP_OPND_IMM;
          step.imm = other->literalAsDouble();
        } else {
          std::array<int64_t, PML_HIP_MAX_RANK> ost{};
          if (!ndStrides(other->shape, out, &ost)) throw std::runtime_error("elementwise operands do not broadcast");
          step.operand_kind = PML_HIP_OPND_TENSOR;
          step.operand = tb.tail.n_operands;
          tb.tail.operand_dtype[tb.tail.n_operands++] = hipType(other->shape.elementType);
          tb.operand_bufs.push_back(bufferFor(other));
          tb.operand_offs.push_back(0);
          tb.nd_strides.push_back(ost);
        }
      } else {
        throw std::runtime_error("elementwise operation '" + op.fn + "' is not supported by the hip target");
      }
      if (step.opcode) tb.tail.ops[tb.tail.n_ops++] = step;
    }
    consumed_.insert(i);
    extendTail(&tb, op.result, i, /*two_d=*/false, /*allow64=*/true);
    for (size_t k = 0; k < tb.nd_strides.size(); ++k)
      std::copy(tb.nd_strides[k].begin(), tb.nd_strides[k].end(), s.elt.operand_strides[k]);
    s.elt.tail = tb.tail;
    s.elt.out_dtype = hipType(tb.final_dtype);
    s.c = bufferFor(tb.final_value);
    attachTail(&s, tb);
    s.text = "eltwise " + (op.kind == Op::Cast ? std::string("cast") : op.fn) + tailText(tb) + " -> " + tb.final_value->shape.str();
    s.bytes = static_cast<double>(out.getByteSize()) * 2;
    plan_->steps.push_back(s);
  }

  // the producer of v if it is a Cast from `from` to v's type
  const Op* castProducer(const ValuePtr& v, DataType from) {
    auto it = producer_.find(v.get());
    if (it == producer_.end()) return nullptr;
    const Op& p = prog_->ops[it->second];
    if (p.kind != Op::Cast || p.operands[0]->shape.elementType != from || p.operands[0]->kind == Value::Literal) return nullptr;
    return &p;
  }

  void emitContraction(size_t i) {
    Op& op = prog_->ops[i];
    if (!op.boundsComputed) tile::computeBounds(&op);
    consumed_.insert(i);
    if (op.result->shape.elements() == 0) return;
    if (opt_.specialise && !emptyBox(op)) {
      if (tryGemm(i)) return;
      if (tryConv(i)) return;
      if (tryDepthwise(i)) return;
      if (tryPool(i)) return;
      if (tryGlobalPool(i)) return;
    }
    emitGeneral(i);
  }

  // fills init_* of a dense kernel from op.init; false if the broadcast pattern is not expressible
  bool denseInit(const Op& op, int32_t* kind, int32_t* dtype, int64_t* rs, int64_t* cs, int* buf) {
    *kind = 0;
    *buf = -1;
    if (!op.init) return true;
    if (op.init->kind == Value::Literal) return false;
    if (!rowColStrides(op.init->shape, op.result->shape, rs, cs)) return false;
    *kind = 1;
    *dtype = hipType(op.init->shape.elementType);
    *buf = bufferFor(op.init);
    return true;
  }

  bool denseTypes(const Op& op, ValuePtr* a, ValuePtr* b, int* in_dt, int* out_dt) {
    const DataType rdt = op.result->shape.elementType;
    *a = op.operands[0];
    *b = op.operands[1];
    const DataType adt = (*a)->shape.elementType, bdt = (*b)->shape.elementType;
    // the matrix-core kernels address an operand with 32-bit byte offsets: larger ones take the general kernel
    const size_t kOffsetLimit = size_t(1) << 31;
    if ((*a)->shape.getByteSize() >= kOffsetLimit || (*b)->shape.getByteSize() >= kOffsetLimit) return false;
    if (adt == bdt && adt == rdt && (rdt == DataType::f32 || rdt == DataType::bf16)) {
      *in_dt = hipType(rdt);
      *out_dt = hipType(rdt);
      return true;
    }
    // cast(A, INT32) (x) cast(B, INT32) with int8 sources: int8 MFMA with int32 accumulation
    if (rdt == DataType::si32 && adt == DataType::si32 && bdt == DataType::si32) {
      const Op* ca = castProducer(*a, DataType::si8);
      const Op* cb = castProducer(*b, DataType::si8);
      if (ca && cb) {
        *a = ca->operands[0];
        *b = cb->operands[0];
        *in_dt = PML_HIP_I8;
        *out_dt = PML_HIP_I32;
        return true;
      }
    }
    return false;
  }

  bool tryGemm(size_t i) {
    const Op& op = prog_->ops[i];
    if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2) return false;
    ValuePtr A, B;
    int in_dt, out_dt;
    if (!denseTypes(op, &A, &B, &in_dt, &out_dt)) return false;
    Normalised n = normalise(op);
    for (const auto& c : n.cons)
      if (!impliedByBox(op, c.lhs, c.rhs)) return false;
    std::vector<int64_t> so, sa, sb;
    int64_t bo, ba, bb;
    if (!indexStrides(n.acc[0], op.result->shape, &so, &bo) || !indexStrides(n.acc[1], op.operands[0]->shape, &sa, &ba) ||
        !indexStrides(n.acc[2], op.operands[1]->shape, &sb, &bb))
      return false;
    // every access must stay in range over the whole box (no padding in a GEMM)
    for (size_t s = 0; s < 3; ++s) {
      const TensorShape& shape = s == 0 ? op.result->shape : op.operands[s - 1]->shape;
      for (size_t d = 0; d < n.acc[s].size(); ++d)
        if (!impliedByBox(op, n.acc[s][d], shape.sizes[d])) return false;
    }
    struct Idx { size_t v; int64_t range, so, sa, sb; };
    std::vector<Idx> M, N, K;
    for (size_t v = 0; v < n.nIdx; ++v) {
      if (!n.active[v]) continue;
      if (op.lower[v] != 0) return false;
      Idx x{v, op.upper[v] + 1, so[v], sa[v], sb[v]};
      const bool o = so[v] != 0, a = sa[v] != 0, b = sb[v] != 0;
      if (o && a && !b) M.push_back(x);
      else if (o && !a && b) N.push_back(x);
      else if (!o && a && b) K.push_back(x);
      else return false;
      if (so[v] < 0 || sa[v] < 0 || sb[v] < 0) return false;
    }
    if (K.empty()) return false;
    // a group collapses to one dimension if, ordered by stride, each stride equals the next stride x range
    auto collapse = [](std::vector<Idx>& g, int64_t Idx::*field, int64_t* ld) {
      std::sort(g.begin(), g.end(), [&](const Idx& x, const Idx& y) { return x.*field > y.*field; });
      for (size_t k = 0; k + 1 < g.size(); ++k)
        if (g[k].*field != g[k + 1].*field * g[k + 1].range) return false;
      *ld = g.empty() ? 0 : g.back().*field;
      return true;
    };
    auto sameOrder = [](const std::vector<Idx>& x, std::vector<Idx> y, int64_t Idx::*field) {
      std::sort(y.begin(), y.end(), [&](const Idx& p, const Idx& q) { return p.*field > q.*field; });
      for (size_t k = 0; k < x.size(); ++k)
        if (x[k].v != y[k].v) return false;
      return true;
    };
    int64_t ldc = 0, lda = 0, ncs = 0, kas = 0, ldb = 0, kbs = 0, nbs = 0;
    if (!collapse(M, &Idx::so, &ldc) || !sameOrder(M, M, &Idx::sa)) return false;
    {
      std::vector<Idx> t = M;
      if (!collapse(t, &Idx::sa, &lda)) return false;
      for (size_t k = 0; k < M.size(); ++k)
        if (t[k].v != M[k].v) return false;
    }
    {
      std::vector<Idx> t = N;
      if (!collapse(N, &Idx::so, &ncs) || !collapse(t, &Idx::sb, &nbs)) return false;
      for (size_t k = 0; k < N.size(); ++k)
        if (t[k].v != N[k].v) return false;
    }
    {
      std::vector<Idx> t = K;
      if (!collapse(K, &Idx::sa, &kas) || !collapse(t, &Idx::sb, &kbs)) return false;
      for (size_t k = 0; k < K.size(); ++k)
        if (t[k].v != K[k].v) return false;
    }
    int64_t m = 1, nn = 1, kk = 1;
    for (const Idx& x : M) m *= x.range;
    for (const Idx& x : N) nn *= x.range;
    for (const Idx& x : K) kk *= x.range;
    // the m x n block must be the whole result: elements the contraction never reaches hold the
    // aggregation identity (or the initial value), which only the general path writes
    if (bo != 0 || m * nn != op.result->shape.elements()) return false;
    if (N.empty()) { ncs = 1; nbs = 1; }   // matrix-vector: one column
    if (M.empty()) { ldc = nn; lda = kk; }  // vector-matrix: one row
    if (ncs != 1 || kas != 1) return false;
    bool b_is_nk;
    if (nbs == 1 || N.empty()) {
      b_is_nk = false;  // B[k][n]
      ldb = kbs;
      if (N.empty()) ldb = std::max<int64_t>(kbs, 1);
      if (ldb < nn) return false;
    } else if (kbs == 1) {
      b_is_nk = true;  // B[n][k]
      ldb = nbs;
      if (ldb < kk) return false;
    } else {
      return false;
    }
    if (ldc < nn || lda < kk) return false;
    const int es = in_dt == PML_HIP_F32 ? 4 : (in_dt == PML_HIP_BF16 ? 2 : 1);
    if ((kk * es) % 16 != 0 || (lda * es) % 16 != 0 || (ba * es) % 16 != 0) return false;
    if (b_is_nk && ((ldb * es) % 16 != 0 || (bb * es) % 16 != 0)) return false;

    Step s;
    s.kind = Step::Gemm;
    pml_hip_gemm_desc& d = s.gemm;
    d.in_dtype = in_dt;
    d.out_dtype = out_dt;
    d.m = m;
    d.n = nn;
    d.k = kk;
    d.lda = lda;
    d.ldb = ldb;
    d.ldc = ldc;
    d.b_layout = b_is_nk ? 1 : 0;
    if (opt_.fp32_as_bf16x3 && in_dt == PML_HIP_F32) d.flags = PML_HIP_FP32_AS_BF16X3;
    if (!denseInit(op, &d.init_kind, &d.init_dtype, &d.init_row_stride, &d.init_col_stride, &s.init)) return false;
    // the tail and the row/col operand addressing assume a dense rows x cols output
    TailBuild tb;
    tb.final_value = op.result;
    tb.final_dtype = op.result->shape.elementType;
    const bool dense_out = ldc == nn && bo == 0 && op.result->shape.getRank() >= 1 && op.result->shape.sizes.back() == nn;
    if (dense_out) extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
    if (d.init_kind && !dense_out && !(d.init_row_stride == 0 && d.init_col_stride <= 1)) return unconsume(tb), false;
    d.tail = tb.tail;
    d.c_dtype = hipType(tb.final_dtype);
    if (tb.tail.n_ops && pml_hip_gemm_tail_cheaper_apart(&d)) {
      // the kernel library multiplies this shape faster under a plain tail: the chain stays with the
      // element-wise operations that follow (which fuse among themselves)
      unconsume(tb);
      tb = TailBuild();
      tb.final_value = op.result;
      tb.final_dtype = op.result->shape.elementType;
      d.tail = tb.tail;
      d.c_dtype = hipType(tb.final_dtype);
    }
    s.a = bufferFor(A);
    s.b = bufferFor(B);
    s.c = bufferFor(tb.final_value);
    s.a_off = ba;
    s.b_off = bb;
    s.c_off = bo;
    s.b_is_nk = b_is_nk;
    s.b_constant = B->kind == Value::Constant;
    attachTail(&s, tb);
    s.flops = 2.0 * m * nn * kk;
    s.bytes = static_cast<double>(m * kk + kk * nn) * es + static_cast<double>(m * nn) * util::byteSize(tb.final_dtype);
    std::stringstream ss;
    ss << "gemm " << util::mnemonic(static_cast<DataType>(in_dt)) << (d.flags & PML_HIP_FP32_AS_BF16X3 ? " (as 3 bf16 products)" : "")
       << " m=" << m << " n=" << nn << " k=" << kk << (b_is_nk ? " B=[n][k]" : " B=[k][n]") << (s.b_constant ? " (constant, packed once)" : "")
       << (d.init_kind ? " +init" : "") << tailText(tb) << " -> " << tb.final_value->shape.str();
    s.text = ss.str();
    plan_->steps.push_back(s);
    return true;
  }

  bool unconsume(const TailBuild& tb) {
    for (size_t c : tb.consumed) consumed_.erase(c);
    return false;
  }

  // spatial form s*x + d*k - p: finds the output index (coef s) and tap index (coef d)
  struct Spatial {
    int out_idx = -1, tap_idx = -1;
    int64_t stride = 1, dil = 1, pad = 0;
  };
  bool spatialForm(const Affine& a, const std::vector<bool>& in_out, const std::vector<bool>& active, Spatial* sp) {
    if (a.den != 1) return false;
    sp->pad = -a.c0;
    for (size_t v = 0; v < a.coef.size(); ++v) {
      if (!a.coef[v]) continue;
      if (!active[v]) return false;
      if (in_out[v]) {
        if (sp->out_idx >= 0) return false;
        sp->out_idx = static_cast<int>(v);
        sp->stride = a.coef[v];
      } else {
        if (sp->tap_idx >= 0) return false;
        sp->tap_idx = static_cast<int>(v);
        sp->dil = a.coef[v];
      }
    }
    return sp->stride > 0 && sp->dil > 0;
  }

  // The output access of a window kernel: every dimension is its own plain index over the whole extent; a
  // dimension of size 1 (batch 1, a 1x1 plane) has had its index folded to the constant 0 and gets index -1.
  bool windowOutput(const Op& op, const Normalised& n, const TensorShape& os, int oi[4], std::vector<bool>* in_out) {
    for (int k = 0; k < 4; ++k) {
      if (os.sizes[k] == 1 && n.acc[0][k].isConstant() && n.acc[0][k].c0 == 0) {
        oi[k] = -1;
        continue;
      }
      oi[k] = n.acc[0][k].plainIndex();
      if (oi[k] < 0 || (*in_out)[oi[k]] || op.lower[oi[k]] != 0 || op.upper[oi[k]] != os.sizes[k] - 1) return false;
      (*in_out)[oi[k]] = true;
    }
    return true;
  }
  // the access form is the index idx, or the constant 0 where that index was folded away (idx < 0)
  static bool sameIndex(const Affine& a, int idx) { return idx >= 0 ? a.plainIndex() == idx : (a.isConstant() && a.c0 == 0); }

  // out[n,y,x,co] += I[n, sy*y + dy*ky - py, sx*x + dx*kx - px, ci] * F[ky,kx,ci,co]
  bool tryConv(size_t i) {
    const Op& op = prog_->ops[i];
    if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2) return false;
    ValuePtr I, F;
    int in_dt, out_dt;
    if (!denseTypes(op, &I, &F, &in_dt, &out_dt)) return false;
    const TensorShape &os = op.result->shape, &is = op.operands[0]->shape, &fs = op.operands[1]->shape;
    if (os.getRank() != 4 || is.getRank() != 4 || fs.getRank() != 4) return false;
    Normalised n = normalise(op);
    for (const auto& c : n.cons)
      if (!impliedByBox(op, c.lhs, c.rhs)) return false;
    // output: four distinct plain indices covering the whole output
    int oi[4];
    std::vector<bool> in_out(n.nIdx, false);
    for (int d = 0; d < 4; ++d) {
      if (os.sizes[d] == 1 && n.acc[0][d].isConstant() && n.acc[0][d].c0 == 0) {
        oi[d] = -1;
        continue;
      }
      oi[d] = n.acc[0][d].plainIndex();
      if (oi[d] < 0 || in_out[oi[d]]) return false;
      if (op.lower[oi[d]] != 0 || op.upper[oi[d]] != os.sizes[d] - 1) return false;
      in_out[oi[d]] = true;
    }
    // input batch and channel
    auto plainOrZero = [&](const Affine& a, int64_t size, int* idx) {
      if (size == 1 && a.isConstant() && a.c0 == 0) {
        *idx = -1;
        return true;
      }
      *idx = a.plainIndex();
      return *idx >= 0;
    };
    int in_n, in_c, f_ci, f_co, f_ky, f_kx;
    if (!plainOrZero(n.acc[1][0], is.sizes[0], &in_n) || in_n != oi[0]) return false;
    if (!plainOrZero(n.acc[1][3], is.sizes[3], &in_c)) return false;
    if (!plainOrZero(n.acc[2][0], fs.sizes[0], &f_ky) || !plainOrZero(n.acc[2][1], fs.sizes[1], &f_kx)) return false;
    if (!plainOrZero(n.acc[2][2], fs.sizes[2], &f_ci) || !plainOrZero(n.acc[2][3], fs.sizes[3], &f_co)) return false;
    if (f_ci != in_c || f_co != oi[3]) return false;
    if (in_c >= 0 && (in_out[in_c] || op.lower[in_c] != 0 || op.upper[in_c] != is.sizes[3] - 1)) return false;
    if (is.sizes[3] != fs.sizes[2] || fs.sizes[3] != os.sizes[3]) return false;
    Spatial sy, sx;
    if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
    if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || sy.tap_idx != f_ky || sx.tap_idx != f_kx) return false;
    if (f_ky >= 0 && (op.lower[f_ky] != 0 || op.upper[f_ky] != fs.sizes[0] - 1)) return false;
    if (f_kx >= 0 && (op.lower[f_kx] != 0 || op.upper[f_kx] != fs.sizes[1] - 1)) return false;
    // every active index must have been given a role
    std::set<int> roles = {oi[0], oi[1], oi[2], oi[3], in_c, f_ky, f_kx};
    for (size_t v = 0; v < n.nIdx; ++v)
      if (n.active[v] && !roles.count(static_cast<int>(v))) return false;
    const int es = in_dt == PML_HIP_F32 ? 4 : (in_dt == PML_HIP_BF16 ? 2 : 1);
    // (channel counts that do not fill 16-byte vectors are handled inside the kernel library: patch matrix + GEMM)

    Step s;
    s.kind = Step::Conv2d;
    pml_hip_conv2d_desc& d = s.conv;
    d.in_dtype = in_dt;
    d.out_dtype = out_dt;
    d.n = is.sizes[0];
    d.h = is.sizes[1];
    d.w = is.sizes[2];
    d.ci = is.sizes[3];
    d.kh = fs.sizes[0];
    d.kw = fs.sizes[1];
    d.co = fs.sizes[3];
    d.oh = os.sizes[1];
    d.ow = os.sizes[2];
    d.stride_h = sy.stride;
    d.stride_w = sx.stride;
    d.dil_h = sy.dil;
    d.dil_w = sx.dil;
    d.pad_h = sy.pad;
    d.pad_w = sx.pad;
    if (opt_.fp32_as_bf16x3 && in_dt == PML_HIP_F32) d.flags = PML_HIP_FP32_AS_BF16X3;
    if (os.sizes[0] != d.n) return false;
    if (!denseInit(op, &d.init_kind, &d.init_dtype, &d.init_row_stride, &d.init_col_stride, &s.init)) return false;
    TailBuild tb;
    extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
    d.tail = tb.tail;
    d.c_dtype = hipType(tb.final_dtype);
    s.a = bufferFor(I);
    s.b = bufferFor(F);
    s.c = bufferFor(tb.final_value);
    s.b_constant = F->kind == Value::Constant;
    attachTail(&s, tb);
    // algorithmic FLOPs: 2 x valid (output, tap) pairs
    auto valid = [](int64_t out, int64_t in, int64_t k, int64_t st, int64_t dl, int64_t pad) {
      int64_t cnt = 0;
      for (int64_t o = 0; o < out; ++o)
        for (int64_t t = 0; t < k; ++t) {
          const int64_t x = o * st + t * dl - pad;
          if (x >= 0 && x < in) ++cnt;
        }
      return cnt;
    };
    s.flops = 2.0 * d.n * valid(d.oh, d.h, d.kh, d.stride_h, d.dil_h, d.pad_h) * valid(d.ow, d.w, d.kw, d.stride_w, d.dil_w, d.pad_w) *
              d.ci * d.co;
    s.bytes = static_cast<double>(is.elements() + fs.elements()) * es + static_cast<double>(os.elements()) * util::byteSize(tb.final_dtype);
    std::stringstream ss;
    ss << "conv2d " << util::mnemonic(static_cast<DataType>(in_dt)) << (d.flags & PML_HIP_FP32_AS_BF16X3 ? " (as 3 bf16 products) " : " ") << is.str() << " (*) " << fs.str() << " stride=" << d.stride_h
       << "x" << d.stride_w << " pad=" << d.pad_h << "," << d.pad_w << (s.b_constant ? " (constant filter, packed once)" : "")
       << (d.init_kind ? " +init" : "") << tailText(tb) << " -> " << tb.final_value->shape.str();
    s.text = ss.str();
    plan_->steps.push_back(s);
    return true;
  }

  // out[n,y,x,c] += I[n, sy*y + dy*ky - py, sx*x + dx*kx - px, c] * F[ky,kx,c,0]
  bool tryDepthwise(size_t i) {
    const Op& op = prog_->ops[i];
    if (op.agg != AggKind::add || op.combo != ComboKind::mul || op.operands.size() != 2 || op.init) return false;
    const DataType dt = op.result->shape.elementType;
    if (dt != DataType::f32 && dt != DataType::bf16) return false;
    if (op.operands[0]->shape.elementType != dt || op.operands[1]->shape.elementType != dt) return false;
    const TensorShape &os = op.result->shape, &is = op.operands[0]->shape, &fs = op.operands[1]->shape;
    if (os.getRank() != 4 || is.getRank() != 4 || fs.getRank() != 4 || fs.sizes[3] != 1) return false;
    Normalised n = normalise(op);
    for (const auto& c : n.cons)
      if (!impliedByBox(op, c.lhs, c.rhs)) return false;
    int oi[4];
    std::vector<bool> in_out(n.nIdx, false);
    if (!windowOutput(op, n, os, oi, &in_out)) return false;
    if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3]) || !sameIndex(n.acc[2][2], oi[3])) return false;
    if (!(n.acc[2][3].isConstant() && n.acc[2][3].c0 == 0)) return false;
    if (is.sizes[3] != os.sizes[3] || fs.sizes[2] != os.sizes[3] || is.sizes[0] != os.sizes[0]) return false;
    Spatial sy, sx;
    if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
    auto tapOk = [&](const Affine& a, int64_t size, int tap) {
      if (size == 1 && a.isConstant() && a.c0 == 0) return tap < 0;
      return a.plainIndex() == tap && tap >= 0 && op.lower[tap] == 0 && op.upper[tap] == size - 1;
    };
    if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || !tapOk(n.acc[2][0], fs.sizes[0], sy.tap_idx) ||
        !tapOk(n.acc[2][1], fs.sizes[1], sx.tap_idx))
      return false;
    std::set<int> roles = {oi[0], oi[1], oi[2], oi[3], sy.tap_idx, sx.tap_idx};
    for (size_t v = 0; v < n.nIdx; ++v)
      if (n.active[v] && !roles.count(static_cast<int>(v))) return false;
    const int V = 16 / static_cast<int>(util::byteSize(dt));
    if (os.sizes[3] % V != 0) return false;
    Step s;
    s.kind = Step::Dwconv2d;
    pml_hip_dwconv2d_desc& d = s.dw;
    d.dtype = hipType(dt);
    d.n = is.sizes[0];
    d.h = is.sizes[1];
    d.w = is.sizes[2];
    d.c = is.sizes[3];
    d.kh = fs.sizes[0];
    d.kw = fs.sizes[1];
    d.oh = os.sizes[1];
    d.ow = os.sizes[2];
    d.stride_h = sy.stride;
    d.stride_w = sx.stride;
    d.dil_h = sy.dil;
    d.dil_w = sx.dil;
    d.pad_h = sy.pad;
    d.pad_w = sx.pad;
    TailBuild tb;
    extendTail(&tb, op.result, i, /*two_d=*/true, /*allow64=*/false);
    if (tb.final_dtype != dt) return unconsume(tb);  // this kernel stores its own element type
    d.tail = tb.tail;
    s.a = bufferFor(op.operands[0]);
    s.b = bufferFor(op.operands[1]);
    s.c = bufferFor(tb.final_value);
    s.b_constant = op.operands[1]->kind == Value::Constant;
    attachTail(&s, tb);
    s.flops = 2.0 * os.elements() * d.kh * d.kw;
    s.bytes = static_cast<double>(is.elements() + os.elements() + fs.elements()) * util::byteSize(dt);
    s.text = "dwconv2d " + std::string(util::mnemonic(dt)) + " " + is.str() + " k=" + std::to_string(d.kh) + "x" + std::to_string(d.kw) +
             " stride=" + std::to_string(d.stride_h) + (s.b_constant ? " (constant filter, packed once)" : "") + tailText(tb) + " -> " +
             tb.final_value->shape.str();
    plan_->steps.push_back(s);
    return true;
  }

  // out[n,y,x,c] = agg I[n, sy*y + ky - py, sx*x + kx - px, c],  ky < KH, kx < KW
  bool poolGeometry(const Op& op, const Normalised& n, pml_hip_pool2d_desc* d, Spatial* sy, Spatial* sx) {
    const TensorShape &os = op.result->shape, &is = op.operands[0]->shape;
    if (os.getRank() != 4 || is.getRank() != 4) return false;
    int oi[4];
    std::vector<bool> in_out(n.nIdx, false);
    if (!windowOutput(op, n, os, oi, &in_out)) return false;
    if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3])) return false;
    if (is.sizes[0] != os.sizes[0] || is.sizes[3] != os.sizes[3]) return false;
    if (!spatialForm(n.acc[1][1], in_out, n.active, sy) || !spatialForm(n.acc[1][2], in_out, n.active, sx)) return false;
    if (sy->out_idx != oi[1] || sx->out_idx != oi[2] || sy->dil != 1 || sx->dil != 1) return false;
    // window extents come from the explicit constraints k < K; a tap index without one is not a pooling window
    int64_t kh = 1, kw = 1;
    bool have_h = sy->tap_idx < 0, have_w = sx->tap_idx < 0;
    for (const auto& c : op.constraints) {
      const int p = c.lhs.plainIndex();
      if (p < 0) return false;
      if (p == sy->tap_idx) {
        kh = c.rhs;
        have_h = true;
      } else if (p == sx->tap_idx) {
        kw = c.rhs;
        have_w = true;
      } else if (!impliedByBox(op, c.lhs, c.rhs)) {
        return false;
      }
    }
    if (!have_h || !have_w) return false;
    d->n = is.sizes[0];
    d->h = is.sizes[1];
    d->w = is.sizes[2];
    d->c = is.sizes[3];
    d->kh = kh;
    d->kw = kw;
    d->oh = os.sizes[1];
    d->ow = os.sizes[2];
    d->stride_h = sy->stride;
    d->stride_w = sx->stride;
    d->pad_h = sy->pad;
    d->pad_w = sx->pad;
    return true;
  }

  // out[n,c] (or out[n,0,0,c]) = agg over all (y,x) of I[n,y,x,c]: a pooling window that is the whole image
  bool tryGlobalPool(size_t i) {
    const Op& op = prog_->ops[i];
    if (op.combo != ComboKind::none || op.operands.size() != 1 || op.init) return false;
    if (op.agg != AggKind::max && op.agg != AggKind::min && op.agg != AggKind::add) return false;
    const DataType dt = op.result->shape.elementType;
    if ((dt != DataType::f32 && dt != DataType::bf16) || op.operands[0]->shape.elementType != dt) return false;
    const TensorShape &os = op.result->shape, &is = op.operands[0]->shape;
    if (is.getRank() != 4) return false;
    const bool keep = os.getRank() == 4;
    if (!keep && os.getRank() != 2) return false;
    if (keep && (os.sizes[1] != 1 || os.sizes[2] != 1)) return false;
    if (os.sizes.front() != is.sizes[0] || os.sizes.back() != is.sizes[3]) return false;
    Normalised n = normalise(op);
    for (const auto& c : n.cons)
      if (!impliedByBox(op, c.lhs, c.rhs)) return false;
    const bool one_image = is.sizes[0] == 1;  // the batch index of a single image is folded to the constant 0
    const int on = one_image ? -1 : n.acc[0].front().plainIndex(), oc = n.acc[0].back().plainIndex();
    if ((!one_image && on < 0) || oc < 0 || on == oc) return false;
    if (one_image && !sameIndex(n.acc[0].front(), -1)) return false;
    if (keep && !(n.acc[0][1].isConstant() && n.acc[0][1].c0 == 0 && n.acc[0][2].isConstant() && n.acc[0][2].c0 == 0)) return false;
    const int iy = n.acc[1][1].plainIndex(), ix = n.acc[1][2].plainIndex();
    if (!sameIndex(n.acc[1][0], on) || n.acc[1][3].plainIndex() != oc || iy < 0 || ix < 0 || iy == ix || iy == on ||
        iy == oc || ix == on || ix == oc)
      return false;
    const int idx[4] = {on, iy, ix, oc};
    for (int k = 0; k < 4; ++k)
      if (idx[k] >= 0 && (op.lower[idx[k]] != 0 || op.upper[idx[k]] != is.sizes[k] - 1)) return false;
    for (size_t v = 0; v < n.nIdx; ++v)
      if (n.active[v] && static_cast<int>(v) != on && static_cast<int>(v) != oc && static_cast<int>(v) != iy &&
          static_cast<int>(v) != ix)
        return false;
    const int V = 16 / static_cast<int>(util::byteSize(dt));
    if (is.sizes[3] % V != 0) return false;
    Step s;
    s.kind = Step::Pool2d;
    pml_hip_pool2d_desc& d = s.pool;
    d.dtype = hipType(dt);
    d.agg = hipAgg(op.agg);
    d.n = is.sizes[0];
    d.h = is.sizes[1];
    d.w = is.sizes[2];
    d.c = is.sizes[3];
    d.kh = d.h;
    d.kw = d.w;
    d.oh = d.ow = 1;
    d.stride_h = d.stride_w = 1;
    d.pad_h = d.pad_w = 0;
    s.a = bufferFor(op.operands[0]);
    s.c = bufferFor(op.result);
    s.bytes = static_cast<double>(is.elements() + os.elements()) * util::byteSize(dt);
    s.text = "pool2d " + tile::toString(op.agg) + " " + std::string(util::mnemonic(dt)) + " " + is.str() +
             " over the whole image -> " + os.str();
    plan_->steps.push_back(s);
    return true;
  }

  bool tryPool(size_t i) {
    const Op& op = prog_->ops[i];
    if (op.combo != ComboKind::none || op.operands.size() != 1 || op.init) return false;
    if (op.agg != AggKind::max && op.agg != AggKind::min && op.agg != AggKind::add) return false;
    const DataType dt = op.result->shape.elementType;
    if ((dt != DataType::f32 && dt != DataType::bf16) || op.operands[0]->shape.elementType != dt) return false;
    Normalised n = normalise(op);
    Step s;
    s.kind = Step::Pool2d;
    Spatial sy, sx;
    if (!poolGeometry(op, n, &s.pool, &sy, &sx)) return false;
    const int V = 16 / static_cast<int>(util::byteSize(dt));
    if (s.pool.c % V != 0) return false;
    s.pool.dtype = hipType(dt);
    s.pool.agg = hipAgg(op.agg);
    s.a = bufferFor(op.operands[0]);
    s.c = bufferFor(op.result);
    // window argmax: AM = max(cond(R[window], M[out], IX[ky,kx])) with IX = ky*KW + kx, same geometry
    if (op.agg == AggKind::max) {
      auto uit = users_.find(op.result.get());
      if (uit != users_.end()) {
        for (size_t ui : uit->second) {
          if (consumed_.count(ui)) continue;
          if (matchWindowArgmax(ui, op, s.pool)) {
            s.pool.with_index = 1;
            s.out2 = bufferFor(prog_->ops[ui].result);
            consumed_.insert(ui);
            break;
          }
        }
      }
    }
    const TensorShape& is = op.operands[0]->shape;
    s.bytes = static_cast<double>(is.elements() + op.result->shape.elements()) * util::byteSize(dt) +
              (s.pool.with_index ? 4.0 * op.result->shape.elements() : 0.0);
    s.text = "pool2d " + tile::toString(op.agg) + " " + std::string(util::mnemonic(dt)) + " " + is.str() + " k=" +
             std::to_string(s.pool.kh) + "x" + std::to_string(s.pool.kw) + " stride=" + std::to_string(s.pool.stride_h) +
             (s.pool.with_index ? " +window argmax" : "") + " -> " + op.result->shape.str();
    plan_->steps.push_back(s);
    return true;
  }

  // IX is (index(dims,0) * KW + index(dims,1)) over dims [KH, KW]
  bool isWindowIota(const ValuePtr& ix, int64_t kh, int64_t kw) {
    if (ix->shape.sizes != std::vector<int64_t>{kh, kw} || ix->shape.elementType != DataType::si32) return false;
    auto prod = [&](const ValuePtr& v) -> const Op* {
      auto it = producer_.find(v.get());
      return it == producer_.end() ? nullptr : &prog_->ops[it->second];
    };
    const Op* add = prod(ix);
    if (!add || add->kind != Op::Eltwise || add->fn != "add" || add->operands.size() != 2) return false;
    for (int side = 0; side < 2; ++side) {
      const Op* mul = prod(add->operands[side]);
      const Op* i1 = prod(add->operands[1 - side]);
      if (!mul || !i1 || i1->kind != Op::Index || i1->axis != 1) continue;
      if (mul->kind != Op::Eltwise || mul->fn != "mul" || mul->operands.size() != 2) continue;
      for (int ms = 0; ms < 2; ++ms) {
        const Op* i0 = prod(mul->operands[ms]);
        const ValuePtr& lit = mul->operands[1 - ms];
        if (i0 && i0->kind == Op::Index && i0->axis == 0 && lit->kind == Value::Literal && !util::isFloat(lit->shape.elementType) &&
            static_cast<int64_t>(lit->literalAsDouble()) == kw)
          return true;
      }
    }
    return false;
  }

  bool matchWindowArgmax(size_t ui, const Op& pool, const pml_hip_pool2d_desc& pd) {
    Op& u = prog_->ops[ui];
    if (u.kind != Op::Contraction || u.agg != AggKind::max || u.combo != ComboKind::cond || u.operands.size() != 3 || u.init) return false;
    if (u.operands[0] != pool.operands[0] || u.operands[1] != pool.result) return false;
    if (u.result->shape.elementType != DataType::si32 || u.result->shape.sizes != pool.result->shape.sizes) return false;
    if (!u.boundsComputed) tile::computeBounds(&u);
    if (emptyBox(u)) return false;
    Normalised n = normalise(u);
    // geometry of the R access must equal the pool's; M access must be the plain output access
    pml_hip_pool2d_desc d{};
    Spatial sy, sx;
    Op probe = u;  // poolGeometry reads operands[0] and explicit constraints only
    // the window extents of this contraction come from IX's shape instead of explicit constraints
    if (n.acc[3].size() != 2) return false;
    const int ky = n.acc[3][0].plainIndex(), kx = n.acc[3][1].plainIndex();
    {
      // re-use the spatial matcher by hand
      std::vector<bool> in_out(n.nIdx, false);
      int oi[4];
      if (!windowOutput(u, n, u.result->shape, oi, &in_out)) return false;
      for (int k = 0; k < 4; ++k)
        if (!sameIndex(n.acc[2][k], oi[k])) return false;
      if (!sameIndex(n.acc[1][0], oi[0]) || !sameIndex(n.acc[1][3], oi[3])) return false;
      if (!spatialForm(n.acc[1][1], in_out, n.active, &sy) || !spatialForm(n.acc[1][2], in_out, n.active, &sx)) return false;
      if (sy.out_idx != oi[1] || sx.out_idx != oi[2] || sy.dil != 1 || sx.dil != 1) return false;
      if (sy.tap_idx != ky || sx.tap_idx != kx) return false;
    }
    (void)probe;
    (void)d;
    if (sy.stride != pd.stride_h || sx.stride != pd.stride_w || sy.pad != pd.pad_h || sx.pad != pd.pad_w) return false;
    if (!u.constraints.empty()) return false;
    return isWindowIota(u.operands[2], pd.kh, pd.kw);
  }

  // ----- the general contraction kernel ---------------------------------------------------

  // Per output dimension the index to solve the output access for, or -1: integer forms only; an index that
  // appears in one output dimension only; among those the widest range (what a thread no longer walks), the
  // smaller coefficient on a tie.  A dimension whose access is a constant keeps -1; if a dimension with indices
  // has no candidate, nothing is solved for (every dimension -1) and the kernel enumerates the whole box.
  static std::vector<int> choosePivots(const Op& op) {
    const size_t nIdx = op.idxNames.size(), rank = op.accesses[0].size();
    std::vector<int> pivot(rank, -1);
    std::vector<int> uses(nIdx, 0);
    for (const Affine& a : op.accesses[0]) {
      if (a.den != 1) return pivot;
      for (size_t v = 0; v < nIdx; ++v) uses[v] += a.coef[v] != 0;
    }
    for (size_t k = 0; k < rank; ++k) {
      const Affine& a = op.accesses[0][k];
      if (a.isConstant()) continue;
      int best = -1;
      for (size_t v = 0; v < nIdx; ++v) {
        if (!a.coef[v] || uses[v] != 1 || std::llabs(a.coef[v]) > (1 << 20)) continue;
        const int64_t range = op.upper[v] - op.lower[v], best_range = best < 0 ? -1 : op.upper[best] - op.lower[best];
        if (best < 0 || range > best_range || (range == best_range && std::llabs(a.coef[v]) < std::llabs(a.coef[best]))) best = static_cast<int>(v);
      }
      if (best < 0) return std::vector<int>(rank, -1);
      pivot[k] = best;
    }
    return pivot;
  }

  void emitGeneral(size_t i) {
    const Op& op = prog_->ops[i];
    const size_t nIdx = op.idxNames.size();
    const TensorShape& os = op.result->shape;
    // output indices: each output dimension is exactly one distinct index (coef 1 or more), den 1
    std::vector<int> out_idx;
    bool injective = true;
    {
      std::set<int> seen;
      for (const Affine& a : op.accesses[0]) {
        if (a.den != 1) {
          injective = false;
          break;
        }
        int found = -1;
        for (size_t v = 0; v < nIdx; ++v) {
          if (!a.coef[v]) continue;
          if (found >= 0) injective = false;
          found = static_cast<int>(v);
        }
        if (found >= 0) {
          if (seen.count(found)) injective = false;
          seen.insert(found);
          out_idx.push_back(found);
        }
      }
    }
    Step s;
    s.kind = Step::Contract;
    pml_hip_contract_desc& d = s.con;
    std::vector<int> order;  // new position -> old index
    std::vector<std::array<int64_t, 2>> extra_box;
    size_t n_fresh = 0;
    // Output accesses that are sums of indices (a transposed convolution's O[n, 2x + i - 1, ...]): the output
    // coordinates o_k become the variables, as in the reference's change of variables
    // (pmlc/dialect/tile/transforms/contraction.cc:340-416, ReduceOutputPolynomials), but one index at a time:
    // in each output dimension one index v -- the one with the widest range among those no other output
    // dimension uses -- is solved for, v = (o_k - the form's other terms) / c, and substituted in every form.
    // Forms then carry the denominator c, and the kernel's "must be an integer" test does what the reference's
    // Defractionalize (:418-561) arranges by a further change of variables; v's own range becomes a constraint.
    // A thread then walks the remaining indices only (the taps and input channels), not the whole box.
    std::vector<int> pivot;  // per output dimension: the index solved for, or -1
    if (injective) {
      order = out_idx;
      d.n_out_idx = static_cast<int>(out_idx.size());
      for (size_t v = 0; v < nIdx; ++v)
        if (std::find(out_idx.begin(), out_idx.end(), static_cast<int>(v)) == out_idx.end()) order.push_back(static_cast<int>(v));
    } else {
      // one fresh index per output dimension, tied to the sink polynomial by an equality form or by solving
      n_fresh = os.getRank();
      d.n_out_idx = static_cast<int>(n_fresh);
      pivot = choosePivots(op);
      for (size_t v = 0; v < nIdx; ++v)
        if (std::find(pivot.begin(), pivot.end(), static_cast<int>(v)) == pivot.end()) order.push_back(static_cast<int>(v));
    }
    const size_t n_solved = pivot.size() - static_cast<size_t>(std::count(pivot.begin(), pivot.end(), -1));
    const size_t total_idx = n_fresh + nIdx - n_solved;
    if (total_idx > PML_HIP_MAX_IDX) throw std::runtime_error("contraction has too many indices for the hip target");
    d.n_idx = static_cast<int>(total_idx);
    d.dtype = hipType(os.elementType);
    d.agg = hipAgg(op.agg);
    d.combo = hipCombo(op.combo);
    d.n_src = static_cast<int>(op.operands.size());
    for (size_t k = 0; k < op.operands.size(); ++k) d.src_dtype[k] = hipType(op.operands[k]->shape.elementType);
    if (op.combo == ComboKind::cond || op.combo == ComboKind::eq)
      d.cmp_dtype = hipType(util::promoteTypes(op.operands[0]->shape.elementType, op.operands[1]->shape.elementType));
    tile::aggregationIdentity(op.agg, os.elementType, &d.identity_f, &d.identity_i);
    // positions: fresh output indices first (non-injective case), then `order`
    std::vector<int> pos(nIdx, -1);
    for (size_t k = 0; k < order.size(); ++k) pos[order[k]] = static_cast<int>(n_fresh + k);
    for (size_t k = 0; k < n_fresh; ++k) {
      d.lo[k] = 0;
      d.hi[k] = os.sizes[k] - 1;
    }
    for (size_t v = 0; v < nIdx; ++v) {
      if (pos[v] < 0) continue;  // solved for
      d.lo[pos[v]] = op.lower[v];
      d.hi[pos[v]] = op.upper[v];
    }
    d.out_elems = 1;
    for (int k = 0; k < d.n_out_idx; ++k) d.out_elems *= std::max<int64_t>(0, d.hi[k] - d.lo[k] + 1);
    int nf = 0;
    // a form over the program's indices -> one over the kernel's (solved indices substituted)
    auto addForm = [&](const Affine& a, int operand, int64_t size, int64_t stride) {
      if (nf >= PML_HIP_MAX_FORMS) throw std::runtime_error("contraction has too many access dimensions for the hip target");
      pml_hip_form& f = d.forms[nf++];
      std::memset(&f, 0, sizeof f);
      // common multiple of the solved indices' coefficients that this form touches
      int64_t scale = 1;
      for (size_t k = 0; k < pivot.size(); ++k)
        if (pivot[k] >= 0 && a.coef[pivot[k]] != 0) scale = std::lcm(scale, std::llabs(op.accesses[0][k].coef[pivot[k]]));
      std::vector<int64_t> coef(total_idx, 0);
      int64_t c0 = a.c0 * scale;
      for (size_t v = 0; v < nIdx; ++v)
        if (pos[v] >= 0) coef[pos[v]] += a.coef[v] * scale;
      for (size_t k = 0; k < pivot.size(); ++k) {
        if (pivot[k] < 0 || a.coef[pivot[k]] == 0) continue;
        const Affine& o = op.accesses[0][k];
        const int64_t m = a.coef[pivot[k]] * (scale / o.coef[pivot[k]]);  // times (o_k - the other terms of o)
        coef[k] += m;
        c0 -= m * o.c0;
        for (size_t w = 0; w < nIdx; ++w)
          if (static_cast<int>(w) != pivot[k] && o.coef[w] != 0) coef[pos[w]] -= m * o.coef[w];
      }
      const int64_t den = a.den * scale;
      for (size_t v = 0; v < total_idx; ++v) {
        if (coef[v] > INT32_MAX || coef[v] < INT32_MIN) throw std::runtime_error("index coefficient too large");
        f.coef[v] = static_cast<int32_t>(coef[v]);
      }
      if (c0 > INT32_MAX || c0 < INT32_MIN || den > INT32_MAX || den <= 0) throw std::runtime_error("index coefficient too large");
      f.c0 = static_cast<int32_t>(c0);
      f.den = static_cast<int32_t>(den);
      f.operand = operand;
      f.size = size;
      f.stride = stride;
      return &f;
    };
    const auto ostr = os.denseStrides();
    if (injective) {
      for (size_t k = 0; k < op.accesses[0].size(); ++k) addForm(op.accesses[0][k], 0, os.sizes[k], ostr[k]);
    } else {
      for (size_t k = 0; k < n_fresh; ++k) {
        // output element = fresh index k; the sink polynomial must equal it: 0 <= sink - o_k < 1
        Affine plain;
        plain.coef.assign(nIdx, 0);
        pml_hip_form* fo = addForm(plain, 0, os.sizes[k], ostr[k]);
        fo->coef[k] = 1;
        const Affine& a = op.accesses[0][k];
        if (pivot[k] >= 0) {
          // the solved index must be an integer of its range: 0 <= v - lower < extent
          Affine v;
          v.coef.assign(nIdx, 0);
          v.coef[pivot[k]] = 1;
          v.c0 = -op.lower[pivot[k]];
          addForm(v, -1, op.upper[pivot[k]] - op.lower[pivot[k]] + 1, 0);
        } else {
          pml_hip_form* fe = addForm(a, -1, 1, 0);
          fe->coef[k] -= static_cast<int32_t>(fe->den);  // (sink_num - den*o_k) / den
        }
      }
    }
    for (size_t sidx = 1; sidx < op.accesses.size(); ++sidx) {
      const TensorShape& sh = op.operands[sidx - 1]->shape;
      const auto st = sh.denseStrides();
      for (size_t k = 0; k < op.accesses[sidx].size(); ++k) {
        const Affine& a = op.accesses[sidx][k];
        // a dimension the box already keeps in range and that contributes nothing can be dropped
        addForm(a, static_cast<int>(sidx), sh.sizes[k], st[k]);
      }
    }
    for (const auto& c : op.constraints) addForm(c.lhs, -1, c.rhs, 0);
    d.n_forms = nf;
    // initial value: the broadcast init tensor, or the identity when some output elements are never written
    int64_t covered = injective ? d.out_elems : 0;
    const bool full_cover = injective && covered == os.elements();
    s.c = bufferFor(op.result);
    if (op.init) {
      d.has_init = 1;
      Step f;
      f.kind = Step::Eltwise;
      f.elt.rank = static_cast<int>(os.getRank());
      if (os.getRank() > PML_HIP_MAX_RANK) throw std::runtime_error("rank > 6 is not supported by the hip target");
      std::array<int64_t, PML_HIP_MAX_RANK> st{};
      if (!ndStrides(op.init->shape, os, &st)) throw std::runtime_error("contraction initialiser does not broadcast to the result");
      for (size_t k = 0; k < os.getRank(); ++k) f.elt.sizes[k] = os.sizes[k];
      std::copy(st.begin(), st.end(), f.elt.in_strides);
      f.elt.in_dtype = hipType(op.init->shape.elementType);
      f.elt.out_dtype = hipType(os.elementType);
      if (op.init->shape.elementType != os.elementType) {
        f.elt.tail.n_ops = 1;
        f.elt.tail.ops[0].opcode = PML_HIP_EPI_CAST;
        f.elt.tail.ops[0].dtype = hipType(os.elementType);
      }
      f.a = bufferFor(op.init);
      f.c = s.c;
      f.text = "broadcast initial value -> " + os.str();
      plan_->steps.push_back(f);
    } else if (!full_cover) {
      d.has_init = 1;
      Step f;
      f.kind = Step::Eltwise;
      f.elt.rank = static_cast<int>(os.getRank());
      for (size_t k = 0; k < os.getRank(); ++k) f.elt.sizes[k] = os.sizes[k];
      f.elt.in_dtype = f.elt.out_dtype = hipType(os.elementType);
      f.a = scalarConstant(os.elementType, d.identity_f, d.identity_i);
      f.c = s.c;
      f.text = "fill with the aggregation identity -> " + os.str();
      plan_->steps.push_back(f);
    }
    for (const ValuePtr& v : op.operands) s.operands.push_back(bufferFor(v));
    std::stringstream ss;
    ss << "contract (general) " << tile::toString(op.agg) << "/" << tile::toString(op.combo) << " idx=" << d.n_idx
       << " out_idx=" << d.n_out_idx;
    if (!injective) {
      ss << " (output enumerated per element";
      if (n_solved) {
        ss << "; solved for";
        for (int v : pivot)
          if (v >= 0) ss << " " << op.idxNames[v];
      }
      ss << ")";
    }
    ss << " -> " << os.str();
    s.text = ss.str();
    plan_->steps.push_back(s);
  }
};

}  // namespace

std::string Plan::dump() const {
  std::stringstream ss;
  ss << "hip plan: " << steps.size() << " launches, " << buffers.size() << " buffers\n";
  for (size_t i = 0; i < steps.size(); ++i) ss << "  [" << i << "] " << steps[i].text << steps[i].schedule << "\n";
  return ss.str();
}

std::shared_ptr<Plan> buildPlan(tile::Program* program, const Options& options) {
  Planner p(program, options);
  return p.run();
}

}  // namespace pmlc::target::hip

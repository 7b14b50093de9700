#include "hip_planner.h"

namespace pmlc::target::hip {

// Two matrix products that are added -- a residual block's projection shortcut and the last 1x1 convolution
// of its main path -- become one launch that accumulates both into the same result tile: the sum is never
// written and read back (the reference reaches the same by fusing the loop nests of producer and consumer,
// pmlc/target/x86/pipeline.cc:304-322).  Works on finished steps: Y = gemm / 1x1 convolution whose tail starts
// with "+ result of X", X = earlier gemm / 1x1 convolution without a tail whose result nobody else reads.
void Planner::fuseSecondProducts() {
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
void Planner::padDepthwiseResults() {
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

// A 3x3 stride-2 max-pool that is the only reader of a convolution's result, where the kernel library's convolution can
// pool its rows before they leave the chip (pml_hip_conv2d_takes_maxpool: the few-channel stride-2 head of an image
// network): the pooling step goes, the convolution writes the pooled tensor, and the full-size result -- 205 MB at
// 128 x 112 x 112 x 64 -- is neither written nor read.  The reference fuses such producer / consumer nests in its own
// way (pmlc/target/x86/pipeline.cc:304-322).  Not under a program-wide convolution path (`hip{conv=...}`).
void Planner::fusePoolIntoConv() {
  if (!opt_.conv.empty()) return;
  for (size_t x = 0; x < plan_->steps.size(); ++x) {
    Step& X = plan_->steps[x];
    if (X.kind != Step::Conv2d || X.c < 0 || X.c_off != 0 || !X.outs.empty() || X.out2 >= 0) continue;
    if (plan_->buffers[X.c].kind != BufferInfo::Temp || PML_HIP_FLAG_MAXPOOL_OF(X.conv.flags)) continue;
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
    const Step& Y = plan_->steps[y];
    const pml_hip_pool2d_desc& q = Y.pool;
    if (Y.kind != Step::Pool2d || Y.a_off != 0 || Y.c < 0 || Y.out2 >= 0 || !Y.outs.empty() || !Y.operands.empty()) continue;
    if (q.agg != PML_HIP_AGG_MAX || q.with_index || q.divisor != 0.f || q.kh != 3 || q.kw != 3 || q.stride_h != 2 || q.stride_w != 2 ||
        q.dtype != PML_HIP_BF16 || q.pad_h < 0 || q.pad_h > 1 || q.pad_w < 0 || q.pad_w > 1)
      continue;
    if (q.n != X.conv.n || q.h != X.conv.oh || q.w != X.conv.ow || q.c != X.conv.co) continue;
    // the padding behind is whatever makes the pooled size come out (taps past the image's end are left out either way)
    int pb = -1, pr = -1;
    for (int e = 1; e >= 0; --e) {
      if ((q.h + q.pad_h + e - 3) / 2 + 1 == q.oh && q.h + q.pad_h + e >= 3) pb = e;
      if ((q.w + q.pad_w + e - 3) / 2 + 1 == q.ow && q.w + q.pad_w + e >= 3) pr = e;
    }
    if (pb < 0 || pr < 0) continue;
    pml_hip_conv2d_desc probe = X.conv;
    probe.flags |= PML_HIP_FLAG_MAXPOOL3x3S2(static_cast<int>(q.pad_h), pb, static_cast<int>(q.pad_w), pr);
    if (!pml_hip_conv2d_takes_maxpool(&probe)) continue;
    X.conv = probe;
    X.c = Y.c;
    X.c_off = Y.c_off;
    const auto arrow = X.text.rfind(" -> ");
    X.text = (arrow == std::string::npos ? X.text : X.text.substr(0, arrow)) + " + max-pool 3x3 stride 2" + Y.text.substr(Y.text.rfind(" -> "));
    X.bytes += Y.bytes - 2.0 * static_cast<double>(q.n * q.h * q.w * q.c) * 2.0;
    plan_->steps.erase(plan_->steps.begin() + y);
  }
}

// A kernel that took over the work of earlier operations (the int8 GEMM reads the un-cast operands, a pool
// kernel also writes the window argmax) can leave launches whose results nobody reads: drop them.
void Planner::pruneDeadSteps() {
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

int Planner::unaryOpcode(const std::string& fn) {
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
void Planner::checkStepType(const std::string& fn, DataType dt) {
  static const std::set<std::string> float_only = {"sin",  "cos",   "tan",   "sinh",  "cosh", "asin", "acos",
                                                   "atan", "asinh", "acosh", "atanh", "erf",  "pow"};
  static const std::set<std::string> int_only = {"bit_and", "bit_or", "bit_xor", "bit_not", "bit_shl", "bit_shr"};
  if (float_only.count(fn) && !util::isFloat(dt))
    throw std::runtime_error("'" + fn + "' needs floating-point operands, got " + util::mnemonic(dt));
  if (int_only.count(fn) && !util::isInteger(dt))
    throw std::runtime_error("'" + fn + "' needs integer operands, got " + util::mnemonic(dt));
}

// opcode when the running value is the first / second operand (0 = not expressible)
int Planner::binaryOpcode(const std::string& fn, bool running_first) {
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
bool Planner::ndStrides(const TensorShape& shape, const TensorShape& out, std::array<int64_t, PML_HIP_MAX_RANK>* st) {
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
bool Planner::rowColStrides(const TensorShape& shape, const TensorShape& out, int64_t* rs, int64_t* cs) {
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
void Planner::extendTail(TailBuild* tb, ValuePtr value, size_t root, bool two_d, bool allow64) {
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

std::string Planner::tailText(const TailBuild& tb) {
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

void Planner::attachTail(Step* s, const TailBuild& tb) {
  s->operands = tb.operand_bufs;
  s->operand_off = tb.operand_offs;
  s->outs = tb.outs;
}

bool Planner::unconsume(const TailBuild& tb) {
  for (size_t c : tb.consumed) consumed_.erase(c);
  return false;
}

}  // namespace pmlc::target::hip

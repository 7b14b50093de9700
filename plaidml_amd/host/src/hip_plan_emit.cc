#include "hip_planner.h"

namespace pmlc::target::hip {

void Planner::emit(size_t i) {
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
void Planner::emitSpecial(size_t i) {
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

void Planner::emitEltwise(size_t i) {
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
const Op* Planner::castProducer(const ValuePtr& v, DataType from) {
  auto it = producer_.find(v.get());
  if (it == producer_.end()) return nullptr;
  const Op& p = prog_->ops[it->second];
  if (p.kind != Op::Cast || p.operands[0]->shape.elementType != from || p.operands[0]->kind == Value::Literal) return nullptr;
  return &p;
}

void Planner::emitContraction(size_t i) {
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
    if (opt_.fuse && trySoftmax(i)) return;
  }
  emitGeneral(i);
}

// Per output dimension the index to solve the output access for, or -1: integer forms only; an index that
// appears in one output dimension only; among those the widest range (what a thread no longer walks), the
// smaller coefficient on a tie.  A dimension whose access is a constant keeps -1; if a dimension with indices
// has no candidate, nothing is solved for (every dimension -1) and the kernel enumerates the whole box.
std::vector<int> Planner::choosePivots(const Op& op) {
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

void Planner::emitGeneral(size_t i) {
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

}  // namespace pmlc::target::hip

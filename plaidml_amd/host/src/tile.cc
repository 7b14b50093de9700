#include "tile.h"

#include <algorithm>
#include <cmath>
#include <functional>
#include <limits>
#include <numeric>
#include <set>
#include <sstream>
#include <unordered_map>

namespace pmlc::tile {

using ast::AffineOp;
using ast::DimNode;
using ast::ExprNode;
using ast::ExprNodePtr;
using ast::PolyNode;
using ast::PolyNodePtr;

std::string toString(AggKind agg) {
  switch (agg) {
    case AggKind::assign: return "assign";
    case AggKind::add: return "add";
    case AggKind::max: return "max";
    case AggKind::min: return "min";
    case AggKind::mul: return "mul";
  }
  return "?";
}
std::string toString(ComboKind combo) {
  switch (combo) {
    case ComboKind::none: return "none";
    case ComboKind::add: return "add";
    case ComboKind::cond: return "cond";
    case ComboKind::eq: return "eq";
    case ComboKind::mul: return "mul";
  }
  return "?";
}

void aggregationIdentity(AggKind agg, DataType dt, double* f, int64_t* i) {
  *f = 0;
  *i = 0;
  if (util::isFloat(dt)) {
    switch (agg) {
      case AggKind::mul: *f = 1.0; break;
      case AggKind::min: *f = std::numeric_limits<double>::infinity(); break;
      case AggKind::max: *f = -std::numeric_limits<double>::infinity(); break;
      default: break;
    }
    return;
  }
  // integers: the 64-bit extreme, then truncated to the element width
  uint64_t bits = 0;
  const bool uns = util::isUnsigned(dt) || dt == DataType::i1;
  switch (agg) {
    case AggKind::mul: bits = 1; break;
    case AggKind::min:
      bits = uns ? std::numeric_limits<uint64_t>::max() : static_cast<uint64_t>(std::numeric_limits<int64_t>::max());
      break;
    case AggKind::max:
      bits = uns ? 0 : static_cast<uint64_t>(std::numeric_limits<int64_t>::min());
      break;
    default: break;
  }
  switch (util::byteSize(dt)) {
    case 1: *i = uns ? static_cast<int64_t>(static_cast<uint8_t>(bits)) : static_cast<int64_t>(static_cast<int8_t>(bits)); break;
    case 2: *i = uns ? static_cast<int64_t>(static_cast<uint16_t>(bits)) : static_cast<int64_t>(static_cast<int16_t>(bits)); break;
    case 4: *i = uns ? static_cast<int64_t>(static_cast<uint32_t>(bits)) : static_cast<int64_t>(static_cast<int32_t>(bits)); break;
    default: *i = static_cast<int64_t>(bits); break;
  }
  if (dt == DataType::i1) *i &= 1;
}

// ---------------------------------------------------------------------------
// rational affine polynomials while walking a PolyNode tree
// ---------------------------------------------------------------------------
namespace {

struct Frac {
  int64_t n = 0, d = 1;
  Frac() = default;
  Frac(int64_t num, int64_t den = 1) : n(num), d(den) { norm(); }  // NOLINT
  void norm() {
    if (d < 0) {
      n = -n;
      d = -d;
    }
    int64_t g = std::gcd(n < 0 ? -n : n, d);
    if (g > 1) {
      n /= g;
      d /= g;
    }
  }
  Frac operator+(const Frac& o) const { return Frac(n * o.d + o.n * d, d * o.d); }
  Frac operator-(const Frac& o) const { return Frac(n * o.d - o.n * d, d * o.d); }
  Frac operator*(const Frac& o) const { return Frac(n * o.n, d * o.d); }
  Frac operator/(const Frac& o) const { return Frac(n * o.d, d * o.n); }
  bool isZero() const { return n == 0; }
};

struct RPoly {
  std::map<uint64_t, Frac> terms;  // index id -> coefficient
  Frac c0;
  bool isConst() const { return terms.empty(); }
};

RPoly combine(const RPoly& a, const RPoly& b, int sign) {
  RPoly r = a;
  for (const auto& kv : b.terms) {
    Frac v = r.terms.count(kv.first) ? r.terms[kv.first] : Frac();
    v = sign > 0 ? v + kv.second : v - kv.second;
    if (v.isZero())
      r.terms.erase(kv.first);
    else
      r.terms[kv.first] = v;
  }
  r.c0 = sign > 0 ? a.c0 + b.c0 : a.c0 - b.c0;
  return r;
}

RPoly scale(const RPoly& a, const Frac& f) {
  RPoly r;
  if (f.isZero()) return r;
  for (const auto& kv : a.terms) r.terms[kv.first] = kv.second * f;
  r.c0 = a.c0 * f;
  return r;
}

struct PolyWalker {
  ast::Evaluator* ev;
  std::vector<uint64_t>* order;            // first-seen order of index ids
  std::map<uint64_t, std::string>* names;  // id -> name

  RPoly walk(const PolyNodePtr& n) {
    switch (n->kind) {
      case PolyNode::Literal: {
        RPoly r;
        r.c0 = Frac(n->value);
        return r;
      }
      case PolyNode::Dim: {
        RPoly r;
        r.c0 = Frac(ev->evaluate(n->dimRef));
        return r;
      }
      case PolyNode::Index: {
        if (std::find(order->begin(), order->end(), n->id) == order->end()) {
          order->push_back(n->id);
          (*names)[n->id] = n->name.empty() ? "x" + std::to_string(order->size() - 1) : n->name;
        }
        RPoly r;
        r.terms[n->id] = Frac(1);
        return r;
      }
      case PolyNode::Op: {
        if (n->op == AffineOp::Neg) return scale(walk(n->operands.at(0)), Frac(-1));
        RPoly a = walk(n->operands.at(0));
        RPoly b = walk(n->operands.at(1));
        switch (n->op) {
          case AffineOp::Add: return combine(a, b, +1);
          case AffineOp::Sub: return combine(a, b, -1);
          case AffineOp::Mul:
            if (b.isConst()) return scale(a, b.c0);
            if (a.isConst()) return scale(b, a.c0);
            throw std::runtime_error("Non-linear polynomial: " + n->str());
          case AffineOp::Div:
            if (!b.isConst() || b.c0.isZero())
              throw std::runtime_error("Divisor of polynomials must be a non-zero constant: " + n->str());
            return scale(a, Frac(1) / b.c0);
          default:
            throw std::runtime_error("max / min are not valid inside an index polynomial");
        }
      }
    }
    throw std::runtime_error("invalid index polynomial");
  }
};

Affine toAffine(const RPoly& p, const std::vector<uint64_t>& order) {
  int64_t den = p.c0.d;
  for (const auto& kv : p.terms) den = std::lcm(den, kv.second.d);
  Affine a;
  a.den = den;
  a.c0 = p.c0.n * (den / p.c0.d);
  a.coef.assign(order.size(), 0);
  for (size_t i = 0; i < order.size(); ++i) {
    auto it = p.terms.find(order[i]);
    if (it != p.terms.end()) a.coef[i] = it->second.n * (den / it->second.d);
  }
  return a;
}

DataType materialise(DataType dt) {
  switch (dt) {
    case DataType::six: return DataType::si32;
    case DataType::uix: return DataType::ui32;
    case DataType::fx: return DataType::f32;
    default: return dt;
  }
}

struct Builder {
  std::shared_ptr<Program> program;
  ast::Evaluator ev;
  std::unordered_map<const ExprNode*, ValuePtr> memo;

  ValuePtr newValue(Value::Kind kind, const TensorShape& shape, const std::string& name = "") {
    auto v = std::make_shared<Value>();
    v->kind = kind;
    v->id = program->nextId++;
    v->shape = shape;
    v->shape.strides.clear();
    v->name = name;
    return v;
  }

  ValuePtr visit(const ExprNodePtr& node) {
    auto it = memo.find(node.get());
    if (it != memo.end()) return it->second;
    ValuePtr v = build(node);
    memo[node.get()] = v;
    return v;
  }

  ValuePtr build(const ExprNodePtr& node) {
    switch (node->kind) {
      case ExprNode::Input:
        throw std::runtime_error("Placeholder '" + node->name + "' is used by the program but is not one of its inputs");
      case ExprNode::ConstTensor: {
        ValuePtr v = newValue(Value::Constant, node->buffer->shape(), node->name);
        v->constant = node->buffer;
        return v;
      }
      case ExprNode::ConstSigned: {
        ValuePtr v = newValue(Value::Literal, TensorShape(DataType::six));
        v->ivalue = node->ivalue;
        return v;
      }
      case ExprNode::ConstUnsigned: {
        ValuePtr v = newValue(Value::Literal, TensorShape(DataType::uix));
        v->uvalue = node->uvalue;
        return v;
      }
      case ExprNode::ConstFloat: {
        ValuePtr v = newValue(Value::Literal, TensorShape(DataType::fx));
        v->fvalue = node->fvalue;
        return v;
      }
      case ExprNode::Dim: {
        ValuePtr v = newValue(Value::Literal, TensorShape(DataType::six));
        v->ivalue = ev.evaluate(node->dimNode);
        return v;
      }
      case ExprNode::Element:
        if (node->expr && node->expr->kind == ExprNode::Intrinsic && node->expr->op == "prng") {
          // the two results of prng are functions of (state, number of values) alone: each becomes an operation
          // of its own, "prng_values" and "prng_state"
          const ExprNodePtr& call = node->expr;
          TensorShape values = ev.getShape(call);
          ValuePtr state = visit(call->operands.at(0));
          if (state->shape.elementType != DataType::ui32 || state->shape.elements() != 3)
            throw std::runtime_error("'prng' needs a state of three ui32 words");
          Op op;
          op.kind = Op::Special;
          op.fn = node->ordinal == 0 ? "prng_values" : "prng_state";
          op.operands = {state};
          op.params = {static_cast<double>(values.elements())};
          op.result = newValue(Value::Temp, ev.getShape(node), call->name);
          program->ops.push_back(op);
          return op.result;
        }
        return visit(node->expr);
      case ExprNode::Pragma:
        return visit(node->expr);
      case ExprNode::Cast: {
        ValuePtr src = visit(node->expr);
        TensorShape shape = ev.getShape(node);
        if (src->kind == Value::Literal) {
          // a cast of a scalar literal is a typed scalar constant
          ValuePtr v = newValue(Value::Literal, TensorShape(node->dtype));
          const DataType st = src->shape.elementType;
          const double d = src->literalAsDouble();
          if (util::isFloat(node->dtype)) {
            v->fvalue = d;
          } else if (util::isFloat(st)) {
            v->ivalue = static_cast<int64_t>(d);
            v->uvalue = static_cast<uint64_t>(d < 0 ? 0 : d);
          } else if (util::isUnsigned(st) || st == DataType::uix) {
            v->uvalue = src->uvalue;
            v->ivalue = static_cast<int64_t>(src->uvalue);
          } else {
            v->ivalue = src->ivalue;
            v->uvalue = static_cast<uint64_t>(src->ivalue);
          }
          return v;
        }
        Op op;
        op.kind = Op::Cast;
        op.operands = {src};
        op.result = newValue(Value::Temp, shape);
        program->ops.push_back(op);
        return op.result;
      }
      case ExprNode::Intrinsic: {
        TensorShape shape = ev.getShape(node);
        shape.elementType = materialise(shape.elementType);
        Op op;
        op.name = node->name;
        if (node->op == "index") {
          op.kind = Op::Index;
          int64_t axis = 0;
          const ExprNodePtr& a = node->operands.at(0);
          if (a->kind == ExprNode::ConstSigned)
            axis = a->ivalue;
          else if (a->kind == ExprNode::ConstUnsigned)
            axis = static_cast<int64_t>(a->uvalue);
          else
            throw std::runtime_error("'index' requires a constant axis");
          if (axis < 0 || axis >= static_cast<int64_t>(shape.getRank())) throw std::runtime_error("'index' axis out of range");
          op.axis = static_cast<int>(axis);
        } else if (node->op == "reshape") {
          op.kind = Op::Reshape;
          ValuePtr src = visit(node->operands.at(0));
          if (src->shape.elements() != shape.elements())
            throw std::runtime_error("'reshape' must preserve the number of elements");
          op.operands = {src};
        } else if (node->op == "shape") {
          // shapes are static here: the extents of the operand as a constant si32 vector
          // (ShapeOpConversion, pmlc/conversion/tile_to_linalg/tile_to_linalg.cc)
          const TensorShape src = ev.getShape(node->operands.at(0));
          auto buf = std::make_shared<util::SimpleBuffer>(shape);
          for (size_t d = 0; d < src.getRank(); ++d) {
            const int32_t extent = static_cast<int32_t>(src.sizes[d]);
            std::memcpy(buf->data() + 4 * d, &extent, 4);
          }
          ValuePtr v = newValue(Value::Constant, shape, "shape");
          v->constant = buf;
          return v;
        } else if (node->op == "prng") {
          throw std::runtime_error("'prng' yields two results: use element(0) for the values and element(1) for the new state");
        } else if (node->op == "gather" || node->op == "scatter" || node->op == "argsort") {
          // tensor operands first, then constants (plaidml/edsl/edsl.h:809-811, 1036-1066, 1645-1690)
          op.kind = Op::Special;
          op.fn = node->op;
          const size_t n_tensors = node->op == "gather" ? 2 : (node->op == "scatter" ? 3 : 1);
          for (size_t k = 0; k < node->operands.size(); ++k) {
            const ExprNodePtr& o = node->operands[k];
            if (k < n_tensors) {
              ValuePtr v = visit(o);
              if (v->kind == Value::Literal) v = materialiseLiteral(v, materialise(v->shape.elementType));
              op.operands.push_back(v);
              continue;
            }
            switch (o->kind) {
              case ExprNode::ConstSigned: op.params.push_back(static_cast<double>(o->ivalue)); break;
              case ExprNode::ConstUnsigned: op.params.push_back(static_cast<double>(o->uvalue)); break;
              case ExprNode::ConstFloat: op.params.push_back(o->fvalue); break;
              case ExprNode::Dim: op.params.push_back(static_cast<double>(ev.evaluate(o->dimNode))); break;
              default: throw std::runtime_error("'" + node->op + "' expects constant arguments after its tensors");
            }
          }
        } else {
          op.kind = Op::Eltwise;
          op.fn = node->op;
          bool all_literal = !node->operands.empty();
          for (const ExprNodePtr& o : node->operands) {
            op.operands.push_back(visit(o));
            all_literal = all_literal && op.operands.back()->kind == Value::Literal;
          }
          // arithmetic on scalar literals only (e.g. the element count a mean divides by) folds to a literal
          if (all_literal) {
            ValuePtr folded = foldLiterals(op.fn, op.operands);
            if (folded) return folded;
          }
        }
        op.result = newValue(Value::Temp, shape, node->name);
        program->ops.push_back(op);
        return op.result;
      }
      case ExprNode::Contraction:
        return buildContraction(node);
    }
    throw std::runtime_error("invalid expression node");
  }

  ValuePtr buildContraction(const ExprNodePtr& node) {
    TensorShape shape = ev.getShape(node);
    Op op;
    op.kind = Op::Contraction;
    op.name = node->name;
    op.agg = node->aggKind;
    op.combo = node->comboKind;
    const size_t want = node->comboKind == ComboKind::none ? 1 : (node->comboKind == ComboKind::cond ? 3 : 2);
    if (node->srcs.size() != want)
      throw std::runtime_error("contraction has " + std::to_string(node->srcs.size()) + " operands, its combination needs " +
                               std::to_string(want));
    // operands first (their sub-graphs are emitted before this op)
    for (const ast::PolyMap& src : node->srcs) {
      ValuePtr v = visit(src.ref);
      if (v->kind == Value::Literal) {
        // a scalar literal operand (e.g. `assign(One())`): materialise as a rank-0 typed constant
        v = materialiseLiteral(v, materialise(v->shape.elementType));
      }
      op.operands.push_back(v);
    }
    if (node->init) {
      op.init = visit(node->init);
      if (op.init->kind == Value::Literal) op.init = materialiseLiteral(op.init, shape.elementType);
    }
    // index variables in first-seen order over sink, sources, constraints (pmlc/ast/builder.cc:311-323)
    std::vector<uint64_t> order;
    std::map<uint64_t, std::string> names;
    PolyWalker walker{&ev, &order, &names};
    std::vector<std::vector<RPoly>> polys;
    {
      std::vector<RPoly> sink;
      if (node->sinkIdxs.size() != shape.getRank()) throw std::runtime_error("contraction output rank mismatch");
      for (const PolyNodePtr& p : node->sinkIdxs) sink.push_back(walker.walk(p));
      polys.push_back(sink);
    }
    for (size_t s = 0; s < node->srcs.size(); ++s) {
      const ast::PolyMap& src = node->srcs[s];
      if (src.idxs.size() != op.operands[s]->shape.getRank())
        throw std::runtime_error("contraction operand #" + std::to_string(s) + " is indexed with " +
                                 std::to_string(src.idxs.size()) + " indices but has rank " +
                                 std::to_string(op.operands[s]->shape.getRank()));
      std::vector<RPoly> acc;
      for (const PolyNodePtr& p : src.idxs) acc.push_back(walker.walk(p));
      polys.push_back(acc);
    }
    std::vector<std::pair<RPoly, int64_t>> cons;
    for (const ast::Constraint& c : node->constraints) cons.emplace_back(walker.walk(c.lhs), ev.evaluate(c.rhs));
    for (uint64_t id : order) op.idxNames.push_back(names[id]);
    for (const auto& acc : polys) {
      std::vector<Affine> forms;
      for (const RPoly& p : acc) forms.push_back(toAffine(p, order));
      op.accesses.push_back(forms);
    }
    for (const auto& c : cons) {
      ConstraintForm cf;
      cf.lhs = toAffine(c.first, order);
      cf.rhs = c.second;
      op.constraints.push_back(cf);
    }
    op.result = newValue(Value::Temp, shape, node->name);
    program->ops.push_back(op);
    return op.result;
  }

  // add / sub / mul / div / neg / max / min of untyped scalar literals; nullptr when not foldable
  ValuePtr foldLiterals(const std::string& fn, const std::vector<ValuePtr>& xs) {
    for (const ValuePtr& x : xs)
      if (!util::isAmbiguous(x->shape.elementType)) return nullptr;
    const bool unary = xs.size() == 1 && fn == "neg";
    if (!unary && xs.size() != 2) return nullptr;
    if (!unary && fn != "add" && fn != "sub" && fn != "mul" && fn != "div" && fn != "max" && fn != "min") return nullptr;
    bool is_float = false, is_unsigned = false;
    for (const ValuePtr& x : xs) {
      is_float = is_float || x->shape.elementType == DataType::fx;
      is_unsigned = is_unsigned || x->shape.elementType == DataType::uix;
    }
    auto asInt = [](const ValuePtr& v) {
      return v->shape.elementType == DataType::uix ? static_cast<int64_t>(v->uvalue) : v->ivalue;
    };
    ValuePtr r = newValue(Value::Literal, TensorShape(is_float ? DataType::fx : (is_unsigned ? DataType::uix : DataType::six)));
    if (is_float) {
      const double a = xs[0]->literalAsDouble(), b = unary ? 0.0 : xs[1]->literalAsDouble();
      r->fvalue = unary ? -a : fn == "add" ? a + b : fn == "sub" ? a - b : fn == "mul" ? a * b : fn == "div" ? a / b
                  : fn == "max" ? std::max(a, b) : std::min(a, b);
    } else {
      const int64_t a = asInt(xs[0]), b = unary ? 0 : asInt(xs[1]);
      if (fn == "div" && b == 0) return nullptr;
      const int64_t v = unary ? -a : fn == "add" ? a + b : fn == "sub" ? a - b : fn == "mul" ? a * b : fn == "div" ? a / b
                        : fn == "max" ? std::max(a, b) : std::min(a, b);
      r->ivalue = v;
      r->uvalue = static_cast<uint64_t>(v);
    }
    return r;
  }

  // turns a scalar literal into a rank-0 host constant of the given type
  ValuePtr materialiseLiteral(const ValuePtr& lit, DataType dt) {
    TensorShape shape(dt);
    auto buf = std::make_shared<util::SimpleBuffer>(shape);
    const double d = lit->literalAsDouble();
    char* p = buf->data();
    switch (dt) {
      case DataType::f32: { float x = static_cast<float>(d); std::memcpy(p, &x, 4); break; }
      case DataType::f64: { std::memcpy(p, &d, 8); break; }
      case DataType::bf16: {
        float x = static_cast<float>(d);
        uint32_t u;
        std::memcpy(&u, &x, 4);
        u += 0x7fffu + ((u >> 16) & 1u);
        uint16_t h = static_cast<uint16_t>(u >> 16);
        std::memcpy(p, &h, 2);
        break;
      }
      case DataType::f16: throw std::runtime_error("float16 scalar constants are not supported");
      default: {
        int64_t v = util::isFloat(lit->shape.elementType) ? static_cast<int64_t>(d)
                    : (lit->shape.elementType == DataType::uix ? static_cast<int64_t>(lit->uvalue) : lit->ivalue);
        std::memcpy(p, &v, util::byteSize(dt));  // little-endian truncation
        break;
      }
    }
    ValuePtr v = newValue(Value::Constant, shape, "cst");
    v->constant = buf;
    return v;
  }
};

std::string affineStr(const Affine& a, const std::vector<std::string>& names) {
  std::stringstream ss;
  bool first = true;
  if (a.den != 1) ss << "(";
  for (size_t i = 0; i < a.coef.size(); ++i) {
    if (!a.coef[i]) continue;
    int64_t c = a.coef[i];
    if (!first) ss << (c < 0 ? " - " : " + ");
    if (first && c < 0) ss << "-";
    if (std::llabs(c) != 1) ss << std::llabs(c) << "*";
    ss << names[i];
    first = false;
  }
  if (a.c0 || first) {
    if (!first) ss << (a.c0 < 0 ? " - " : " + ");
    if (first && a.c0 < 0) ss << "-";
    ss << std::llabs(a.c0);
  }
  if (a.den != 1) ss << ") / " << a.den;
  return ss.str();
}

std::string valueRef(const ValuePtr& v) {
  switch (v->kind) {
    case Value::Input: return "%arg" + std::to_string(v->id);
    case Value::Constant: return "%cst" + std::to_string(v->id);
    case Value::Literal: {
      std::stringstream ss;
      if (v->shape.elementType == DataType::fx || util::isFloat(v->shape.elementType))
        ss << v->fvalue;
      else if (v->shape.elementType == DataType::uix || util::isUnsigned(v->shape.elementType))
        ss << v->uvalue;
      else
        ss << v->ivalue;
      ss << " : " << util::mnemonic(v->shape.elementType);
      return ss.str();
    }
    case Value::Temp: return "%" + std::to_string(v->id);
  }
  return "?";
}

}  // namespace

std::string Program::str() const {
  std::stringstream ss;
  ss << "module @" << name << " {\n  func @main(";
  for (size_t i = 0; i < inputs.size(); ++i)
    ss << (i ? ", " : "") << valueRef(inputs[i]) << ": tensor<" << inputs[i]->shape.str() << ">";
  ss << ") -> (";
  for (size_t i = 0; i < outputs.size(); ++i) ss << (i ? ", " : "") << "tensor<" << outputs[i]->shape.str() << ">";
  ss << ") {\n";
  for (const Op& op : ops) {
    ss << "    " << valueRef(op.result) << " = ";
    switch (op.kind) {
      case Op::Contraction: {
        ss << "tile.contract " << toString(op.agg) << ", " << toString(op.combo) << ", ";
        ss << (op.init ? valueRef(op.init) : std::string("identity"));
        for (const ValuePtr& v : op.operands) ss << ", " << valueRef(v);
        ss << " {idxs = [";
        for (size_t i = 0; i < op.idxNames.size(); ++i) ss << (i ? ", " : "") << op.idxNames[i];
        ss << "], sink = (";
        for (size_t d = 0; d < op.accesses[0].size(); ++d) ss << (d ? ", " : "") << affineStr(op.accesses[0][d], op.idxNames);
        ss << "), srcs = [";
        for (size_t s = 1; s < op.accesses.size(); ++s) {
          ss << (s > 1 ? ", (" : "(");
          for (size_t d = 0; d < op.accesses[s].size(); ++d) ss << (d ? ", " : "") << affineStr(op.accesses[s][d], op.idxNames);
          ss << ")";
        }
        ss << "]";
        if (!op.constraints.empty()) {
          ss << ", cons = [";
          for (size_t c = 0; c < op.constraints.size(); ++c)
            ss << (c ? ", " : "") << "0 <= " << affineStr(op.constraints[c].lhs, op.idxNames) << " < " << op.constraints[c].rhs;
          ss << "]";
        }
        if (op.boundsComputed) {
          ss << ", lowerBounds = (";
          for (size_t i = 0; i < op.lower.size(); ++i) ss << (i ? ", " : "") << op.lower[i];
          ss << "), upperBounds = (";
          for (size_t i = 0; i < op.upper.size(); ++i) ss << (i ? ", " : "") << op.upper[i];
          ss << ")";
        }
        ss << "}";
        break;
      }
      case Op::Eltwise:
        ss << "tile." << op.fn;
        for (size_t i = 0; i < op.operands.size(); ++i) ss << (i ? ", " : " ") << valueRef(op.operands[i]);
        break;
      case Op::Cast:
        ss << "tile.cast " << valueRef(op.operands[0]);
        break;
      case Op::Index:
        ss << "tile.index " << op.axis;
        break;
      case Op::Reshape:
        ss << "tile.reshape " << valueRef(op.operands[0]);
        break;
      case Op::Special:
        ss << "tile." << op.fn;
        for (size_t i = 0; i < op.operands.size(); ++i) ss << (i ? ", " : " ") << valueRef(op.operands[i]);
        ss << " {";
        for (size_t i = 0; i < op.params.size(); ++i) ss << (i ? ", " : "") << op.params[i];
        ss << "}";
        break;
    }
    ss << " : tensor<" << op.result->shape.str() << ">\n";
  }
  ss << "    return";
  for (size_t i = 0; i < outputs.size(); ++i) ss << (i ? ", " : " ") << valueRef(outputs[i]);
  ss << "\n  }\n}\n";
  return ss.str();
}

std::shared_ptr<Program> buildProgram(const std::string& name, const std::vector<ExprNodePtr>& inputs,
                                      const std::vector<ExprNodePtr>& outputs) {
  Builder b;
  b.program = std::make_shared<Program>();
  b.program->name = name;
  for (const ExprNodePtr& in : inputs) {
    if (!in || in->kind != ExprNode::Input) throw std::runtime_error("program inputs must be Placeholders");
    for (int64_t d : in->shape.sizes)
      if (d <= 0) throw std::runtime_error("Placeholder '" + in->name + "' has an unknown dimension; static shapes are required");
    ValuePtr v = b.newValue(Value::Input, in->shape, in->name);
    b.memo[in.get()] = v;
    b.program->inputs.push_back(v);
  }
  for (const ExprNodePtr& out : outputs) {
    ValuePtr v = b.visit(out);
    if (v->kind == Value::Literal) v = b.materialiseLiteral(v, materialise(v->shape.elementType));
    b.program->outputs.push_back(v);
  }
  b.program->passes.emplace_back("tile", b.program->str());
  return b.program;
}

void eliminateDeadOps(Program* program) {
  std::set<const Value*> live;
  for (const ValuePtr& v : program->outputs) live.insert(v.get());
  std::vector<Op> kept;
  for (auto it = program->ops.rbegin(); it != program->ops.rend(); ++it) {
    if (!live.count(it->result.get())) continue;
    for (const ValuePtr& v : it->operands) live.insert(v.get());
    if (it->init) live.insert(it->init.get());
    kept.push_back(*it);
  }
  std::reverse(kept.begin(), kept.end());
  program->ops = kept;
}

void foldAddIntoInit(Program* program) {
  // use counts
  std::map<const Value*, int> uses;
  for (const Op& op : program->ops) {
    for (const ValuePtr& v : op.operands) uses[v.get()]++;
    if (op.init) uses[op.init.get()]++;
  }
  for (const ValuePtr& v : program->outputs) uses[v.get()]++;
  std::map<const Value*, size_t> producer;
  for (size_t i = 0; i < program->ops.size(); ++i) producer[program->ops[i].result.get()] = i;
  for (size_t i = 0; i < program->ops.size(); ++i) {
    Op& add = program->ops[i];
    if (add.kind != Op::Eltwise || add.fn != "add" || add.operands.size() != 2) continue;
    for (int side = 0; side < 2; ++side) {
      const ValuePtr& c = add.operands[side];
      const ValuePtr& b = add.operands[1 - side];
      auto it = producer.find(c.get());
      if (it == producer.end()) continue;
      Op& con = program->ops[it->second];
      if (con.kind != Op::Contraction || con.agg != AggKind::add || con.init) continue;
      if (uses[c.get()] != 1) continue;
      if (b->kind != Value::Input && b->kind != Value::Constant) continue;
      if (b->shape.elementType != c->shape.elementType || add.result->shape != c->shape) continue;
      if (b->shape.getRank() > c->shape.getRank()) continue;
      // the add takes over the contraction: same result value, contraction gets the initial value
      Op merged = con;
      merged.init = b;
      merged.result = add.result;
      merged.result->name = con.result->name;
      // keep program order valid: place the merged op where the add was, drop the original
      program->ops[i] = merged;
      program->ops[it->second].kind = Op::Eltwise;
      program->ops[it->second].fn = "<dead>";
      program->ops[it->second].operands.clear();
      program->ops[it->second].init.reset();
      break;
    }
  }
  program->ops.erase(std::remove_if(program->ops.begin(), program->ops.end(),
                                    [](const Op& op) { return op.kind == Op::Eltwise && op.fn == "<dead>"; }),
                     program->ops.end());
}

static int64_t floorDiv(int64_t a, int64_t b) {
  int64_t q = a / b, r = a % b;
  return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

// ---------------------------------------------------------------------------------------------------------------
// Bounds of a contraction's index variables (reference: Contraction::ComputeBounds and Constraints::ComputeBounds,
// pmlc/dialect/tile/transforms/contraction.cc:107-149,657-681, which minimise and maximise every variable with an
// integer linear program, pmlc/util/bilp).  The valid set is
//     { integer x : for every form f:  (coef_f . x + c0_f) / den_f  is an integer in [0, size_f) }
// over all accesses (output and inputs) and all constraints.  Three steps, each sound on its own:
//   1. interval propagation: every form bounds each of its variables from the bounds of the others;
//   2. where that leaves a variable unbounded (a domain bounded only by combinations of forms, e.g. 0 <= i + j < 10
//      together with 0 <= i - j < 10), Fourier-Motzkin elimination of the other variables from the linear
//      relaxation gives its range, and propagation runs again from there;
//   3. exact tightening: a bound is moved inwards while no integer point of the set takes that value, decided by a
//      depth-first search over the remaining variables with propagation at every node (the integrality of
//      fractional forms is checked at the leaves).  The search has a node budget; on exhausting it the bounds stay
//      as they are -- still a superset, and the kernels check every form at every point anyway.
// ---------------------------------------------------------------------------------------------------------------
namespace {

constexpr int64_t kInfBound = static_cast<int64_t>(1) << 60;

struct BoundForm {
  const Affine* a;
  int64_t size;
};

// One pass structure of step 1; returns false when some variable's range becomes empty.
bool propagateBounds(const std::vector<BoundForm>& forms, std::vector<int64_t>& lo, std::vector<int64_t>& hi) {
  const size_t n = lo.size();
  for (int iter = 0; iter < 256; ++iter) {
    bool changed = false;
    for (const BoundForm& f : forms) {
      // 0 <= sum coef*idx + c0 <= den*(size-1)
      const int64_t loRhs = -f.a->c0, hiRhs = f.a->den * (f.size - 1) - f.a->c0;
      for (size_t v = 0; v < n; ++v) {
        const int64_t c = f.a->coef[v];
        if (!c) continue;
        int64_t restLo = 0, restHi = 0;
        bool finite = true;
        for (size_t u = 0; u < n && finite; ++u) {
          if (u == v || !f.a->coef[u]) continue;
          if (lo[u] <= -kInfBound || hi[u] >= kInfBound) {
            finite = false;
            break;
          }
          const int64_t a = f.a->coef[u] * lo[u], b = f.a->coef[u] * hi[u];
          restLo += std::min(a, b);
          restHi += std::max(a, b);
        }
        if (!finite) continue;
        const int64_t a = loRhs - restHi, b = hiRhs - restLo;
        int64_t nlo, nhi;
        if (c > 0) {
          nlo = -floorDiv(-a, c);
          nhi = floorDiv(b, c);
        } else {
          nlo = -floorDiv(-b, c);
          nhi = floorDiv(a, c);
        }
        if (nlo > lo[v]) {
          lo[v] = nlo;
          changed = true;
        }
        if (nhi < hi[v]) {
          hi[v] = nhi;
          changed = true;
        }
        if (lo[v] > hi[v]) return false;
      }
    }
    if (!changed) break;
  }
  return true;
}

// Step 2.  Rows are inequalities  sum a[v] * x[v] + a[n] >= 0  with integer coefficients.
typedef std::vector<__int128> IneqRow;

void normaliseRow(IneqRow& r) {
  __int128 g = 0;
  for (size_t i = 0; i + 1 < r.size(); ++i) {
    __int128 x = r[i] < 0 ? -r[i] : r[i];
    while (x) {
      const __int128 t = g % x;
      g = x;
      x = t;
    }
  }
  if (g > 1) {
    for (size_t i = 0; i + 1 < r.size(); ++i) r[i] /= g;
    // floor of the constant: the left-hand side is an integer multiple of g
    __int128 c = r.back();
    __int128 q = c / g;
    if (c % g != 0 && c < 0) --q;
    r.back() = q;
  }
}

// Range of variable `keep` in the linear relaxation: 1 = found, 0 = unbounded on either side, -1 = no range found after
// the elimination grew past its budget of rows.  Past the budget the rows with the most variables are dropped: fewer
// constraints describe a larger set, so a range found then still contains the true one (the integer search that
// follows tightens it), it is only no longer the relaxation's own.  `order` picks the elimination order: 0 = the variable that makes the fewest new rows
// first, 1 = by index, 2 = by index from the back, 3 = no elimination chain at all, only pairs of forms over the kept variable and one other
// (further tries when the first runs out of budget).
int fourierMotzkinRange(const std::vector<BoundForm>& forms, size_t n, size_t keep, int64_t* lo, int64_t* hi, int order = 0) {
  std::set<IneqRow> rows;
  for (const BoundForm& f : forms) {
    IneqRow up(n + 1), down(n + 1);
    for (size_t v = 0; v < n; ++v) {
      up[v] = f.a->coef[v];
      down[v] = -f.a->coef[v];
    }
    up[n] = f.a->c0;
    down[n] = static_cast<__int128>(f.a->den) * (f.size - 1) - f.a->c0;
    normaliseRow(up);
    normaliseRow(down);
    rows.insert(up);
    rows.insert(down);
  }
  const size_t kBudget = 1500;
  int prunings = 0;
  bool pruned = false;
  if (order == 3) {
    // last try, a relaxation that stays small: for every other variable u, only the rows over {keep, u}, and only u
    // eliminated -- pairs of forms such as a x + b u and a x - b u bound x whatever else the system holds
    pruned = true;
    std::set<IneqRow> single;
    auto support_in = [&](const IneqRow& r, size_t u) {
      for (size_t i = 0; i < n; ++i)
        if (i != keep && i != u && r[i] != 0) return false;
      return true;
    };
    for (size_t u = 0; u < n; ++u) {
      if (u == keep) continue;
      std::vector<const IneqRow*> pos, neg;
      for (const IneqRow& r : rows) {
        if (!support_in(r, u)) continue;
        if (r[u] > 0) pos.push_back(&r);
        else if (r[u] < 0) neg.push_back(&r);
        else if (r[keep] != 0) single.insert(r);
      }
      for (const IneqRow* p : pos)
        for (const IneqRow* q : neg) {
          IneqRow r(n + 1);
          const __int128 cp = (*p)[u], cq = -(*q)[u];
          for (size_t i = 0; i <= n; ++i) r[i] = cq * (*p)[i] + cp * (*q)[i];
          if (r[keep] == 0) continue;
          normaliseRow(r);
          single.insert(r);
        }
    }
    rows.swap(single);
  }
  std::vector<bool> gone(n, false);
  for (size_t step = 0; step + 1 < n && order != 3; ++step) {
    // the variable whose elimination makes the fewest new rows
    size_t best = n;
    size_t bestCost = 0;
    for (size_t k = 0; k < n; ++k) {
      const size_t v = order == 2 ? n - 1 - k : k;
      if (v == keep || gone[v]) continue;
      if (order == 1 || order == 2) {
        best = v;
        break;
      }
      size_t pos = 0, neg = 0;
      for (const IneqRow& r : rows) {
        if (r[v] > 0) ++pos;
        if (r[v] < 0) ++neg;
      }
      const size_t cost = pos * neg;
      if (best == n || cost < bestCost) {
        best = v;
        bestCost = cost;
      }
    }
    if (best == n) break;
    std::set<IneqRow> next;
    std::vector<const IneqRow*> pos, neg;
    for (const IneqRow& r : rows) {
      if (r[best] > 0)
        pos.push_back(&r);
      else if (r[best] < 0)
        neg.push_back(&r);
      else
        next.insert(r);
    }
    for (const IneqRow* p : pos)
      for (const IneqRow* q : neg) {
        IneqRow r(n + 1);
        const __int128 cp = (*p)[best], cq = -(*q)[best];
        for (size_t i = 0; i <= n; ++i) r[i] = cq * (*p)[i] + cp * (*q)[i];
        bool any = false;
        for (size_t i = 0; i < n; ++i) any = any || r[i] != 0;
        if (!any) continue;  // a statement about constants only
        normaliseRow(r);
        next.insert(r);
        if (next.size() > 2 * kBudget) {
          if (++prunings > 4) return -1;
          pruned = true;
          std::vector<std::pair<size_t, IneqRow>> ranked;
          for (const IneqRow& row : next) {
            size_t vars = 0;
            for (size_t i = 0; i < n; ++i) vars += row[i] != 0;
            ranked.emplace_back(vars, row);
          }
          std::stable_sort(ranked.begin(), ranked.end(), [](const auto& x, const auto& y) { return x.first < y.first; });
          next.clear();
          for (size_t i = 0; i < kBudget; ++i) next.insert(ranked[i].second);
        }
      }
    rows.swap(next);
    gone[best] = true;
  }
  bool haveLo = false, haveHi = false;
  __int128 vlo = 0, vhi = 0;
  for (const IneqRow& r : rows) {
    bool only = true;
    for (size_t i = 0; i < n; ++i)
      if (i != keep && r[i] != 0) only = false;
    if (!only || r[keep] == 0) continue;
    // a * x + c >= 0
    const __int128 a = r[keep], c = r[n];
    if (a > 0) {  // x >= ceil(-c / a)
      __int128 q = (-c) / a;
      if ((-c) % a != 0 && (-c) > 0) ++q;
      if (!haveLo || q > vlo) vlo = q;
      haveLo = true;
    } else {  // x <= floor(c / -a)
      const __int128 d = -a;
      __int128 q = c / d;
      if (c % d != 0 && c < 0) --q;
      if (!haveHi || q < vhi) vhi = q;
      haveHi = true;
    }
  }
  if (!haveLo || !haveHi) return pruned ? -1 : 0;
  if (vlo < -kInfBound / 2 || vhi > kInfBound / 2) return pruned ? -1 : 0;
  *lo = static_cast<int64_t>(vlo);
  *hi = static_cast<int64_t>(vhi);
  return 1;
}

// Step 3: is there an integer point of the set inside the box?  `budget` counts search nodes; -1 = gave up.
int feasiblePoint(const std::vector<BoundForm>& forms, std::vector<int64_t> lo, std::vector<int64_t> hi, int64_t* budget) {
  if (--*budget < 0) return -1;
  if (!propagateBounds(forms, lo, hi)) return 0;
  const size_t n = lo.size();
  // branch on the open variable with the smallest range
  size_t pick = n;
  for (size_t v = 0; v < n; ++v) {
    if (lo[v] == hi[v]) continue;
    if (pick == n || hi[v] - lo[v] < hi[pick] - lo[pick]) pick = v;
  }
  if (pick == n) {
    for (const BoundForm& f : forms) {
      __int128 num = f.a->c0;
      for (size_t v = 0; v < n; ++v) num += static_cast<__int128>(f.a->coef[v]) * lo[v];
      if (num < 0 || num % f.a->den != 0 || num / f.a->den >= f.size) return 0;
    }
    return 1;
  }
  // values from the middle outwards: interior points are the likeliest to be valid
  const int64_t mid = lo[pick] + (hi[pick] - lo[pick]) / 2;
  for (int64_t d = 0; mid - d >= lo[pick] || mid + d <= hi[pick]; ++d) {
    for (int side = 0; side < (d ? 2 : 1); ++side) {
      const int64_t x = side ? mid + d : mid - d;
      if (x < lo[pick] || x > hi[pick]) continue;
      std::vector<int64_t> l2 = lo, h2 = hi;
      l2[pick] = h2[pick] = x;
      const int r = feasiblePoint(forms, l2, h2, budget);
      if (r != 0) return r;
    }
  }
  return 0;
}

}  // namespace

void computeBounds(Op* op) {
  if (op->kind != Op::Contraction) return;
  const size_t n = op->idxNames.size();
  std::vector<int64_t> lo(n, -kInfBound), hi(n, kInfBound);
  std::vector<BoundForm> forms;
  for (size_t s = 0; s < op->accesses.size(); ++s) {
    const TensorShape& shape = s == 0 ? op->result->shape : op->operands[s - 1]->shape;
    for (size_t d = 0; d < op->accesses[s].size(); ++d) forms.push_back({&op->accesses[s][d], shape.sizes[d]});
  }
  for (const ConstraintForm& c : op->constraints) forms.push_back({&c.lhs, c.rhs});
  auto emptySet = [&]() {
    // no valid index tuple at all: an empty box (the result is the initial value)
    for (size_t v = 0; v < n; ++v) {
      lo[v] = 0;
      hi[v] = -1;
    }
  };
  bool nonEmpty = propagateBounds(forms, lo, hi);
  if (nonEmpty) {
    bool open = false;
    for (size_t v = 0; v < n; ++v) open = open || lo[v] <= -kInfBound || hi[v] >= kInfBound;
    if (open) {
      for (size_t v = 0; v < n; ++v) {
        if (lo[v] > -kInfBound && hi[v] < kInfBound) continue;
        int64_t l = 0, h = 0;
        int found = -1;
        for (int order = 0; order < 4 && found < 0; ++order) found = fourierMotzkinRange(forms, n, v, &l, &h, order);
        if (found < 0)
          throw std::runtime_error("Bounds too complex: eliminating the other indices around '" + op->idxNames[v] + "' of contraction '" +
                                   op->name + "' outgrows the budget of inequalities in every order tried");
        if (found == 0)
          throw std::runtime_error("Unbounded index '" + op->idxNames[v] + "' in contraction '" + op->name + "'");
        lo[v] = std::max(lo[v], l);
        hi[v] = std::min(hi[v], h);
      }
      nonEmpty = propagateBounds(forms, lo, hi);
    }
  }
  if (nonEmpty) {
    // exact tightening (step 3), within a budget of search nodes for the whole contraction
    int64_t budget = 200000;
    bool gaveUp = false, empty = false;
    for (size_t v = 0; v < n && !gaveUp && !empty; ++v) {
      for (int side = 0; side < 2 && !gaveUp && !empty; ++side) {
        for (;;) {
          if (lo[v] > hi[v]) {
            empty = true;
            break;
          }
          std::vector<int64_t> l2 = lo, h2 = hi;
          l2[v] = h2[v] = side ? hi[v] : lo[v];
          const int r = feasiblePoint(forms, l2, h2, &budget);
          if (r < 0) {
            gaveUp = true;
            break;
          }
          if (r > 0) break;
          if (side)
            --hi[v];
          else
            ++lo[v];
        }
      }
    }
    if (empty) nonEmpty = false;
  }
  if (!nonEmpty) emptySet();
  op->lower = lo;
  op->upper = hi;
  op->boundsComputed = true;
}

void computeBounds(Program* program) {
  for (Op& op : program->ops) computeBounds(&op);
}

}  // namespace pmlc::tile

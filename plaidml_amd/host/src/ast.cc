#include "ast.h"

#include <algorithm>
#include <set>
#include <sstream>

namespace pmlc::ast {

static const char* affineOpStr(AffineOp op) {
  switch (op) {
    case AffineOp::Neg: return "neg";
    case AffineOp::Add: return "add";
    case AffineOp::Sub: return "sub";
    case AffineOp::Mul: return "mul";
    case AffineOp::Div: return "div";
    case AffineOp::Max: return "max";
    case AffineOp::Min: return "min";
  }
  return "?";
}

std::string DimNode::str() const {
  switch (kind) {
    case None: return "?";
    case Literal: return std::to_string(value);
    case Ref: return "dim(" + (ref ? ref->str() : std::string("null")) + ", " + std::to_string(dim) + ")";
    case Op: {
      std::stringstream ss;
      ss << affineOpStr(op) << "(";
      for (size_t i = 0; i < operands.size(); ++i) ss << (i ? ", " : "") << operands[i]->str();
      ss << ")";
      return ss.str();
    }
  }
  return "?";
}

std::string PolyNode::str() const {
  switch (kind) {
    case Dim: return dimRef->str();
    case Index: return name.empty() ? "x" + std::to_string(id) : name;
    case Literal: return std::to_string(value);
    case Op: {
      std::stringstream ss;
      ss << affineOpStr(op) << "(";
      for (size_t i = 0; i < operands.size(); ++i) ss << (i ? ", " : "") << operands[i]->str();
      ss << ")";
      return ss.str();
    }
  }
  return "?";
}

std::string ExprNode::str() const {
  switch (kind) {
    case Input: return name.empty() ? "input" : name;
    case ConstTensor: return name.empty() ? "constant" : name;
    case ConstSigned: return std::to_string(ivalue);
    case ConstUnsigned: return std::to_string(uvalue);
    case ConstFloat: {
      std::stringstream ss;
      ss << fvalue;
      return ss.str();
    }
    case Cast: return std::string("cast(") + expr->str() + ", " + util::mnemonic(dtype) + ")";
    case Contraction: return name.empty() ? "contraction" : name;
    case Dim: return dimNode->str();
    case Element: return expr->str() + "[" + std::to_string(ordinal) + "]";
    case Pragma: return op + "(" + expr->str() + ")";
    case Intrinsic: {
      std::stringstream ss;
      ss << op << "(";
      for (size_t i = 0; i < operands.size(); ++i) ss << (i ? ", " : "") << operands[i]->str();
      ss << ")";
      return ss.str();
    }
  }
  return "?";
}

bool isCompareOp(const std::string& fn) {
  static const std::set<std::string> s = {"cmp_eq", "cmp_ne", "cmp_lt", "cmp_gt", "cmp_le", "cmp_ge"};
  return s.count(fn) != 0;
}
bool isLogicalOp(const std::string& fn) {
  static const std::set<std::string> s = {"logical_and", "logical_or", "logical_not", "logical_xor"};
  return s.count(fn) != 0;
}
bool isKnownIntrinsic(const std::string& fn) {
  static const std::set<std::string> s = {
      "abs",     "add",     "sub",     "mul",      "div",      "mod",     "neg",     "ident",   "relu",   "exp",
      "log",     "sqrt",    "tanh",    "floor",    "ceil",     "round",   "pow",     "sin",     "cos",    "tan",
      "sinh",    "cosh",    "erf",     "select",   "index",    "reshape", "shape",   "bit_and", "bit_or", "bit_xor",
      "bit_not", "bit_shl", "bit_shr", "acos",     "asin",     "atan",    "acosh",   "asinh",   "atanh",
      "gather",  "scatter", "argsort", "prng"};
  return s.count(fn) != 0 || isCompareOp(fn) || isLogicalOp(fn);
}

static bool mergeShapes(TensorShape* into, const TensorShape& from, DataType override_dtype) {
  const auto& a = into->sizes;
  const auto& b = from.sizes;
  std::vector<int64_t> result = a.size() > b.size() ? a : b;
  auto ia = a.rbegin(), ib = b.rbegin();
  auto ir = result.rbegin();
  for (; ia != a.rend() && ib != b.rend(); ++ia, ++ib, ++ir) {
    if (*ia == *ib || *ib == 1) {
      *ir = *ia;
    } else if (*ia == 1) {
      *ir = *ib;
    } else {
      return false;
    }
  }
  DataType dt = override_dtype;
  if (dt == DataType::invalid) dt = util::promoteTypes(into->elementType, from.elementType);
  *into = TensorShape(dt, result);
  return true;
}

TensorShape inferShape(const std::vector<TensorShape>& operands, DataType override_dtype) {
  if (operands.empty()) throw std::runtime_error("operation without operands");
  TensorShape ret = operands.front();
  ret.strides.clear();
  if (override_dtype != DataType::invalid) ret.elementType = override_dtype;
  for (size_t i = 1; i < operands.size(); ++i) {
    if (!mergeShapes(&ret, operands[i], override_dtype)) {
      std::stringstream ss;
      ss << "Incompatible types: (";
      for (size_t j = 0; j < operands.size(); ++j) ss << (j ? ", " : "") << operands[j].str();
      ss << ")";
      throw std::runtime_error(ss.str());
    }
  }
  return ret;
}

static bool integerOperand(Evaluator* ev, const ExprNodePtr& n, int64_t* out) {
  switch (n->kind) {
    case ExprNode::ConstSigned: *out = n->ivalue; return true;
    case ExprNode::ConstUnsigned: *out = static_cast<int64_t>(n->uvalue); return true;
    case ExprNode::Dim: *out = ev->evaluate(n->dimNode); return true;
    default: return false;
  }
}

int64_t Evaluator::evaluate(const DimNodePtr& node) {
  if (!node) throw std::runtime_error("null TensorDim");
  switch (node->kind) {
    case DimNode::Literal:
      return node->value;
    case DimNode::None:
      throw std::runtime_error("DimNodeNone cannot be evaluated: the TensorDim was never bound");
    case DimNode::Ref: {
      TensorShape shape = getShape(node->ref);
      if (node->dim >= shape.getRank()) throw std::runtime_error("TensorDim refers to a missing dimension");
      return shape.sizes[node->dim];
    }
    case DimNode::Op: {
      if (node->op == AffineOp::Neg) return -evaluate(node->operands.at(0));
      const int64_t lhs = evaluate(node->operands.at(0));
      const int64_t rhs = evaluate(node->operands.at(1));
      switch (node->op) {
        case AffineOp::Add: return lhs + rhs;
        case AffineOp::Sub: return lhs - rhs;
        case AffineOp::Mul: return lhs * rhs;
        case AffineOp::Div:
          if (rhs == 0) throw std::runtime_error("division of a TensorDim by zero");
          return lhs / rhs;
        case AffineOp::Max: return std::max(lhs, rhs);
        case AffineOp::Min: return std::min(lhs, rhs);
        default: break;
      }
      throw std::runtime_error("invalid TensorDim operation");
    }
  }
  throw std::runtime_error("invalid TensorDim");
}

TensorShape Evaluator::getShape(const ExprNodePtr& node) {
  if (!node) throw std::runtime_error("null tensor expression");
  auto it = cache_.find(node.get());
  if (it != cache_.end()) return it->second;
  TensorShape shape = computeShape(node);
  cache_.emplace(node.get(), shape);
  return shape;
}

TensorShape Evaluator::computeShape(const ExprNodePtr& node) {
  switch (node->kind) {
    case ExprNode::Input:
      return node->shape;
    case ExprNode::ConstTensor: {
      TensorShape s = node->buffer->shape();
      return s;
    }
    case ExprNode::ConstSigned:
      return TensorShape(DataType::six);
    case ExprNode::ConstUnsigned:
      return TensorShape(DataType::uix);
    case ExprNode::ConstFloat:
      return TensorShape(DataType::fx);
    case ExprNode::Dim:
      return TensorShape(DataType::six);
    case ExprNode::Cast: {
      TensorShape s = getShape(node->expr);
      return TensorShape(node->dtype, s.sizes);
    }
    case ExprNode::Element:
      // prng is the one intrinsic with two results: the values and the advanced state (pmlc/ast/ast_ops.cc:180-195)
      if (node->expr && node->expr->kind == ExprNode::Intrinsic && node->expr->op == "prng") {
        if (node->ordinal == 0) return getShape(node->expr);
        if (node->ordinal == 1) return getShape(node->expr->operands.at(0));
        throw std::runtime_error("'prng' has two results");
      }
      if (node->ordinal != 0) throw std::runtime_error("only single-result expressions are supported");
      return getShape(node->expr);
    case ExprNode::Pragma:
      return getShape(node->expr);
    case ExprNode::Contraction: {
      // result element type: eq -> i1, cond -> type of the third operand, else the promoted operand type
      DataType dt = DataType::invalid;
      if (node->comboKind == ComboKind::eq) {
        dt = DataType::i1;
      } else if (node->comboKind == ComboKind::cond) {
        if (node->srcs.size() != 3) throw std::runtime_error("'cond' contraction needs three operands");
        dt = getShape(node->srcs[2].ref).elementType;
      } else {
        for (const PolyMap& src : node->srcs) dt = util::promoteTypes(dt, getShape(src.ref).elementType);
      }
      if (util::isAmbiguous(dt)) throw std::runtime_error("'contraction' operand data type is ambiguous, use a cast");
      TensorShape s(dt);
      for (const DimNodePtr& d : node->sinkDims) s.sizes.push_back(evaluate(d));
      return s;
    }
    case ExprNode::Intrinsic: {
      std::vector<TensorShape> shapes;
      for (const ExprNodePtr& o : node->operands) shapes.push_back(getShape(o));
      const std::string& fn = node->op;
      if (isCompareOp(fn) || isLogicalOp(fn)) return inferShape(shapes, DataType::i1);
      if (fn == "index") {
        if (node->operands.size() < 2) throw std::runtime_error("'index' requires an axis operand and at least 1 dimension");
        TensorShape ret(DataType::si32);
        for (size_t i = 1; i < node->operands.size(); ++i) {
          int64_t v;
          if (!integerOperand(this, node->operands[i], &v))
            throw std::runtime_error("Additional parameters to 'index' must be integers or TensorDims.");
          ret.sizes.push_back(v);
        }
        return ret;
      }
      if (fn == "reshape") {
        if (node->operands.empty()) throw std::runtime_error("'reshape' requires at least one argument.");
        TensorShape ret(shapes[0].elementType);
        for (size_t i = 1; i < node->operands.size(); ++i) {
          int64_t v;
          if (!integerOperand(this, node->operands[i], &v))
            throw std::runtime_error("Additional parameters to 'reshape' must be integers or TensorDims.");
          ret.sizes.push_back(v);
        }
        return ret;
      }
      if (fn == "prng") {
        // the shape of the first result; operands: the state, then the dims of the values
        if (node->operands.empty()) throw std::runtime_error("'prng' requires at least one argument.");
        TensorShape ret(DataType::f32);
        for (size_t i = 1; i < node->operands.size(); ++i) {
          int64_t v;
          if (!integerOperand(this, node->operands[i], &v))
            throw std::runtime_error("'prng' has invalid operands, dims must be tensor dimensions");
          ret.sizes.push_back(v);
        }
        return ret;
      }
      // the special operations: pmlc/ast/ast_ops.cc:41-60 (argsort), :88-178 (gather), :219-257 (scatter)
      if (fn == "argsort") {
        if (node->operands.size() != 3) throw std::runtime_error("'argsort' requires 3 arguments.");
        int64_t v;
        if (!integerOperand(this, node->operands[1], &v)) throw std::runtime_error("'argsort' requires operand #2 to be an integer.");
        if (!integerOperand(this, node->operands[2], &v)) throw std::runtime_error("'argsort' requires operand #3 to be an integer.");
        return TensorShape(DataType::si32, shapes[0].sizes);
      }
      if (fn == "gather") {
        if (node->operands.size() != 9) throw std::runtime_error("'gather' requires nine arguments.");
        const TensorShape& tensor = shapes[0];
        const TensorShape& idxs = shapes[1];
        const int64_t rank = static_cast<int64_t>(tensor.getRank());
        if (!rank) throw std::runtime_error("'gather' requires first operand to have at least one dimension.");
        int64_t axis, interp, nearest, mode, batch_dims, oob;
        if (!integerOperand(this, node->operands[2], &axis) || axis >= rank || axis < 0)
          throw std::runtime_error(
              "'gather' primitive expects the 'axis' argument to be a positive integer that is less than the tensor rank.");
        if (!integerOperand(this, node->operands[3], &interp))
          throw std::runtime_error("'gather' primitive expects the 'interpolationMode' argument to be a constant integer");
        if (!integerOperand(this, node->operands[4], &nearest))
          throw std::runtime_error("'gather' primitive expects the 'nearestMode' argument to be a constant integer");
        if (node->operands[5]->kind != ExprNode::ConstFloat)
          throw std::runtime_error("'gather' primitive expects the 'cubeCoeff' argument to be a constant float");
        if (!integerOperand(this, node->operands[6], &mode))
          throw std::runtime_error("'gather' primitive expects the 'mode' argument to be a constant integer");
        if (mode == 1 && !util::isInteger(idxs.elementType))
          throw std::runtime_error("'gather' ND mode requires indices elements to be integers.");
        if (!integerOperand(this, node->operands[7], &batch_dims))
          throw std::runtime_error("'gather' primitive expects the 'batchDims' argument to be a constant integer");
        if (!integerOperand(this, node->operands[8], &oob))
          throw std::runtime_error("'gather' primitive expects the 'outOfBoundsMode' argument to be a constant integer");
        TensorShape shape(tensor.elementType);
        if (mode == 0) {
          for (int64_t i = 0; i < axis; ++i) shape.sizes.push_back(tensor.sizes[i]);
          shape.sizes.insert(shape.sizes.end(), idxs.sizes.begin(), idxs.sizes.end());
          for (int64_t i = axis + 1; i < rank; ++i) shape.sizes.push_back(tensor.sizes[i]);
        } else {
          if (idxs.getRank() == 0) throw std::runtime_error("'gather' ND mode requires indices of at least one dimension.");
          for (size_t i = 0; i + 1 < idxs.getRank(); ++i) shape.sizes.push_back(idxs.sizes[i]);
          for (int64_t i = idxs.sizes.back() + batch_dims; i < rank; ++i) shape.sizes.push_back(tensor.sizes[i]);
        }
        return shape;
      }
      if (fn == "scatter") {
        if (node->operands.size() != 5) throw std::runtime_error("'scatter' requires 5 operands.");
        const int64_t rank = static_cast<int64_t>(shapes[0].getRank());
        if (!rank) throw std::runtime_error("'scatter' requires operand #1 to have at least one dimension.");
        if (shapes[1].elementType != DataType::si32 && shapes[1].elementType != DataType::ui32)
          throw std::runtime_error("'scatter' requires operand #2 to be an integer.");
        int64_t axis, mode;
        if (!integerOperand(this, node->operands[3], &axis) || axis >= rank)
          throw std::runtime_error(
              "'scatter' primitive expects the 'axis' argument to be a positive integer that is less than the updates tensor rank.");
        if (!integerOperand(this, node->operands[4], &mode))
          throw std::runtime_error("'scatter' primitive expects the 'mode' argument to be a constant integer.");
        return TensorShape(shapes[0].elementType, shapes[0].sizes);
      }
      if (fn == "shape") {
        if (node->operands.size() != 1) throw std::runtime_error("'shape' requires exactly one argument.");
        return TensorShape(DataType::si32, {static_cast<int64_t>(shapes[0].getRank())});
      }
      if (fn == "select") {
        if (shapes.size() != 3) throw std::runtime_error("'select' requires three operands");
        TensorShape s = inferShape(shapes);
        DataType dt = util::promoteTypes(shapes[1].elementType, shapes[2].elementType);
        if (util::isAmbiguous(dt)) throw std::runtime_error("'select' has ambiguous operand types, use a cast");
        if (shapes[1].elementType != dt || shapes[2].elementType != dt)
          throw std::runtime_error("'select' has unmatched operand types, use a cast");
        return TensorShape(dt, s.sizes);
      }
      if (!isKnownIntrinsic(fn)) throw std::runtime_error("unknown intrinsic '" + fn + "'");
      return inferShape(shapes);
    }
  }
  throw std::runtime_error("invalid expression node");
}

void Evaluator::bindDims(const ExprNodePtr& node, std::vector<DimNodePtr*> into) {
  TensorShape shape = getShape(node);
  if (into.size() != shape.getRank()) throw std::runtime_error("Rank mismatch in bind_dims");
  bool failed = false;
  for (size_t i = 0; i < into.size(); ++i) {
    DimNodePtr* ptr = into[i];
    const int64_t dim = shape.sizes[i];
    switch ((*ptr)->kind) {
      case DimNode::None:
      case DimNode::Ref: {
        auto lit = std::make_shared<DimNode>(DimNode::Literal);
        lit->value = dim;
        *ptr = lit;
        break;
      }
      case DimNode::Literal:
        if (dim != (*ptr)->value) failed = true;
        break;
      default:
        throw std::runtime_error("Can only bind dims to an unbound or previously bound TensorDim.");
    }
  }
  if (failed) {
    std::stringstream s1, s2;
    for (size_t i = 0; i < shape.sizes.size(); ++i) s1 << (i ? ", " : "") << shape.sizes[i];
    for (size_t i = 0; i < into.size(); ++i) {
      s2 << (i ? ", " : "");
      if ((*into[i])->kind == DimNode::Literal)
        s2 << (*into[i])->value;
      else
        s2 << '?';
    }
    throw std::runtime_error("bind dims mismatch: shape=[" + s1.str() + "] != dims=[" + s2.str() + "]");
  }
}

}  // namespace pmlc::ast

// The lowered form of a program: a list of Tile operations over values, the
// role the `tile` dialect module plays in the reference (tile.contract:
// pmlc/dialect/tile/ir/ops.td:20-83; elementwise ops: ir/eltwise.td:119-172).
// Built from the AST by ProgramBuilder (pmlc/ast/builder.cc:303-624 restated),
// then annotated by the bounds pass (pmlc/dialect/tile/transforms/contraction.cc).
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <vector>

#include "ast.h"
#include "util.h"

namespace pmlc::tile {

using ast::AggKind;
using ast::ComboKind;
using util::DataType;
using util::TensorShape;

// (sum_i coef[i] * idx[i] + c0) / den over the index variables of one contraction
struct Affine {
  std::vector<int64_t> coef;  // one per index variable
  int64_t c0 = 0;
  int64_t den = 1;
  bool isConstant() const {
    for (int64_t c : coef)
      if (c) return false;
    return true;
  }
  // the single index this form equals (coef 1, no constant, den 1), or -1
  int plainIndex() const {
    if (den != 1 || c0 != 0) return -1;
    int found = -1;
    for (size_t i = 0; i < coef.size(); ++i) {
      if (coef[i] == 0) continue;
      if (coef[i] != 1 || found >= 0) return -1;
      found = static_cast<int>(i);
    }
    return found;
  }
};

struct Value {
  enum Kind { Input, Constant, Literal, Temp } kind = Temp;
  int id = 0;
  TensorShape shape;
  std::string name;
  util::BufferPtr constant;  // Constant
  // Literal: scalar constants of the program text (dtype six / uix / fx until materialised)
  int64_t ivalue = 0;
  uint64_t uvalue = 0;
  double fvalue = 0;
  double literalAsDouble() const {
    if (shape.elementType == DataType::fx || util::isFloat(shape.elementType)) return fvalue;
    if (shape.elementType == DataType::uix || util::isUnsigned(shape.elementType)) return static_cast<double>(uvalue);
    return static_cast<double>(ivalue);
  }
};
using ValuePtr = std::shared_ptr<Value>;

struct ConstraintForm {
  Affine lhs;
  int64_t rhs = 0;  // 0 <= lhs < rhs
};

struct Op {
  enum Kind { Contraction, Eltwise, Cast, Index, Reshape, Special } kind = Eltwise;
  ValuePtr result;
  std::vector<ValuePtr> operands;
  std::string name;
  // Eltwise
  std::string fn;
  // Index
  int axis = 0;
  // Special (fn = gather / scatter / argsort): the tensor operands are in `operands`, the constant arguments here
  // in the order the intrinsic takes them
  std::vector<double> params;
  // Contraction
  AggKind agg = AggKind::assign;
  ComboKind combo = ComboKind::none;
  std::vector<std::string> idxNames;
  std::vector<std::vector<Affine>> accesses;  // [0] = sink, [1..] = sources (parallel to operands)
  std::vector<ConstraintForm> constraints;
  ValuePtr init;  // optional
  // filled by computeBounds: inclusive box per index
  std::vector<int64_t> lower, upper;
  bool boundsComputed = false;
};

struct Program {
  std::string name;
  std::vector<ValuePtr> inputs;
  std::vector<ValuePtr> outputs;
  std::vector<Op> ops;
  std::vector<std::pair<std::string, std::string>> passes;  // (pass name, text after it)
  std::string target;
  std::shared_ptr<void> compiled;  // the target's plan, set by compile()
  int nextId = 0;
  std::string str() const;
};

// AST -> Program.  `inputs` must be ExprNode::Input nodes; every Input reachable
// from `outputs` has to be listed.
std::shared_ptr<Program> buildProgram(const std::string& name, const std::vector<ast::ExprNodePtr>& inputs,
                                      const std::vector<ast::ExprNodePtr>& outputs);

// `contraction(add) + B` -> contraction(add, init = B)
// (AddInitPattern, pmlc/dialect/tile/transforms/algebraic_opt.cc:30-75)
void foldAddIntoInit(Program* program);

// Per-index inclusive bounds of every contraction by interval propagation over
// all access and constraint forms.  Throws if an index is unbounded.  The valid
// index set is still decided per tuple by the forms, so the box only has to
// contain it (role of Contraction::ComputeBounds,
// pmlc/dialect/tile/transforms/contraction.cc:657-681).
void computeBounds(Program* program);
void computeBounds(Op* op);

// removes operations whose results are unused
void eliminateDeadOps(Program* program);

// aggregation identity narrowed to the element type
// (pmlc/dialect/tile/ir/util.cc:217-260 then the narrowing of tile_to_linalg.cc:85-87)
void aggregationIdentity(AggKind agg, DataType dt, double* f, int64_t* i);

std::string toString(AggKind agg);
std::string toString(ComboKind combo);

}  // namespace pmlc::tile

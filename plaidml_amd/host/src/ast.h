// The expression tree the EDSL builds through the C ABI, and its shape / dtype
// inference.  Restates pmlc/ast/{ast.h:27-373, eval.cc:22-362, ast_ops.cc} of the
// reference (nodes are immutable once built; handles in the C ABI wrap shared_ptrs).
#pragma once

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "util.h"

namespace pmlc::ast {

using util::DataType;
using util::TensorShape;

enum class AffineOp { Neg, Add, Sub, Mul, Div, Max, Min };
enum class AggKind { assign, add, max, min, mul };     // pmlc/util/enums.td:9-19
enum class ComboKind { none, add, cond, eq, mul };     // pmlc/util/enums.td:21-33

struct ExprNode;
using ExprNodePtr = std::shared_ptr<ExprNode>;

// ---- dimension expressions ---------------------------------------------------
struct DimNode {
  enum Kind { None, Literal, Op, Ref } kind;
  int64_t value = 0;                              // Literal
  AffineOp op = AffineOp::Add;                    // Op
  std::vector<std::shared_ptr<DimNode>> operands; // Op
  ExprNodePtr ref;                                // Ref: size of dimension `dim` of `ref`
  size_t dim = 0;
  explicit DimNode(Kind k) : kind(k) {}
  std::string str() const;
};
using DimNodePtr = std::shared_ptr<DimNode>;

// ---- index polynomials -------------------------------------------------------
struct PolyNode {
  enum Kind { Dim, Index, Literal, Op } kind;
  DimNodePtr dimRef;                               // Dim
  std::string name;                                // Index
  uint64_t id = 0;                                 // Index: identity of the variable
  int64_t value = 0;                               // Literal
  AffineOp op = AffineOp::Add;                     // Op
  std::vector<std::shared_ptr<PolyNode>> operands; // Op
  explicit PolyNode(Kind k) : kind(k) {}
  std::string str() const;
};
using PolyNodePtr = std::shared_ptr<PolyNode>;

struct PolyMap {
  ExprNodePtr ref;
  std::vector<PolyNodePtr> idxs;
};
struct Constraint {
  PolyNodePtr lhs;
  DimNodePtr rhs;
};

// ---- tensor expressions ------------------------------------------------------
struct ExprNode {
  enum Kind { Input, ConstTensor, ConstSigned, ConstUnsigned, ConstFloat, Cast, Contraction, Dim, Element, Intrinsic, Pragma };
  Kind kind;
  std::string name;
  // Input
  TensorShape shape;
  // ConstTensor
  util::BufferPtr buffer;
  // scalar constants
  int64_t ivalue = 0;
  uint64_t uvalue = 0;
  double fvalue = 0;
  // Cast
  DataType dtype = DataType::invalid;
  // Cast / Element / Pragma: operand
  ExprNodePtr expr;
  size_t ordinal = 0;
  // Contraction
  AggKind aggKind = AggKind::assign;
  ComboKind comboKind = ComboKind::none;
  std::vector<DimNodePtr> sinkDims;
  std::vector<PolyNodePtr> sinkIdxs;
  std::vector<PolyMap> srcs;
  std::vector<Constraint> constraints;
  ExprNodePtr init;
  // Dim
  DimNodePtr dimNode;
  // Intrinsic
  std::string op;
  std::vector<ExprNodePtr> operands;
  // Pragma
  std::map<std::string, std::string> attrs;

  explicit ExprNode(Kind k) : kind(k) {}
  std::string str() const;
};

// Shape and dtype inference with memoisation; one evaluator per query is cheap.
class Evaluator {
 public:
  TensorShape getShape(const ExprNodePtr& node);
  int64_t evaluate(const DimNodePtr& node);
  void bindDims(const ExprNodePtr& node, std::vector<DimNodePtr*> into);
  void verify(const ExprNodePtr& node) { (void)getShape(node); }

 private:
  TensorShape computeShape(const ExprNodePtr& node);
  std::unordered_map<const ExprNode*, TensorShape> cache_;
};

// numpy-style broadcast of operand shapes with dtype promotion (pmlc/ast/eval.cc:46-136)
TensorShape inferShape(const std::vector<TensorShape>& operands, DataType override_dtype = DataType::invalid);

// the registered elementwise / special intrinsic names (pmlc/dialect/tile/ir/eltwise.td:119-172)
bool isCompareOp(const std::string& fn);
bool isLogicalOp(const std::string& fn);
bool isKnownIntrinsic(const std::string& fn);

}  // namespace pmlc::ast

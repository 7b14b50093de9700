// Definitions of the opaque handle types of the C ABI: each wraps a shared_ptr to
// the real object so that clones are cheap aliases
// (reference: plaidml/core/internal.h:16-34).
#pragma once

#include <atomic>
#include <memory>
#include <sstream>
#include <string>
#include <vector>

#include "ast.h"
#include "hip_runtime.h"
#include "plaidml/core/ffi.h"
#include "plaidml/edsl/ffi.h"
#include "plaidml/exec/ffi.h"
#include "plaidml/op/ffi.h"
#include "tile.h"
#include "util.h"

extern "C" {

struct plaidml_string {
  std::string str;
};
struct plaidml_shape {
  pmlc::util::TensorShape shape;
};
struct plaidml_buffer {
  pmlc::util::BufferPtr buffer;
};
struct plaidml_dim_expr {
  pmlc::ast::DimNodePtr node;
};
struct plaidml_poly_expr {
  pmlc::ast::PolyNodePtr node;
};
struct plaidml_expr {
  pmlc::ast::ExprNodePtr node;
};
struct plaidml_program {
  std::shared_ptr<pmlc::tile::Program> program;
};
struct plaidml_executable {
  std::shared_ptr<pmlc::tile::Program> program;  // kept alive for shape checks at run time
  std::unique_ptr<pmlc::rt::Executable> exec;
};
struct plaidml_value {
  plaidml_value_kind kind = PLAIDML_VALUE_NONE;
  pmlc::ast::DimNodePtr dim;
  pmlc::ast::ExprNodePtr expr;
  double f = 0;
  int64_t i = 0;
  std::string s;
  std::vector<std::shared_ptr<plaidml_value>> tuple;
  std::string str() const {
    std::stringstream ss;
    switch (kind) {
      case PLAIDML_VALUE_NONE: ss << "None"; break;
      case PLAIDML_VALUE_DIM: ss << dim->str(); break;
      case PLAIDML_VALUE_EXPR: ss << expr->str(); break;
      case PLAIDML_VALUE_FLOAT: ss << f; break;
      case PLAIDML_VALUE_INT: ss << i; break;
      case PLAIDML_VALUE_STR: ss << "'" << s << "'"; break;
      case PLAIDML_VALUE_TUPLE:
        ss << "(";
        for (size_t k = 0; k < tuple.size(); ++k) ss << (k ? ", " : "") << tuple[k]->str();
        ss << ")";
        break;
    }
    return ss.str();
  }
};

}  // extern "C"

// The Tile EDSL for C++: TensorDim, TensorIndex, Tensor, Contraction and the
// elementwise intrinsics, with the names and call shapes of the reference header
// (plaidml/edsl/edsl.h:83-1768) so that existing Tile programs compile as they
// are.  Everything is a thin handle over the C ABI (plaidml/edsl/ffi.h).
//
// Not provided (outside the contraction hot path): gather, scatter, argsort, prng
// and the trigonometric intrinsics other than tanh.
#pragma once

#include <algorithm>
#include <functional>
#include <memory>
#include <ostream>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

#include "plaidml/core/core.h"
#include "plaidml/edsl/ffi.h"

namespace plaidml {
namespace edsl {

class Contraction;
class IndexedTensor;
class Tensor;
class TensorDim;
class TensorIndex;
class Value;
struct Constraint;

inline void init() {
  plaidml::init();
  ffi::call_void(plaidml_edsl_init);
}

inline std::vector<std::string> list_targets() {
  auto strs = ffi::own(ffi::call<plaidml_strings*>(plaidml_targets_get), plaidml_strings_free);
  std::vector<std::string> ret;
  for (size_t i = 0; i < strs->size; ++i) ret.push_back(ffi::str(strs->elts[i]));
  return ret;
}

// ---- TensorDim: a symbolic tensor dimension -----------------------------------
class TensorDim {
 public:
  TensorDim() : ptr_(wrap(ffi::call<plaidml_dim_expr*>(plaidml_dim_expr_none))) {}
  explicit TensorDim(const std::shared_ptr<plaidml_dim_expr>& ptr) : ptr_(ptr) {}
  explicit TensorDim(int64_t value) : ptr_(wrap(ffi::call<plaidml_dim_expr*>(plaidml_dim_expr_int, value))) {}
  TensorDim(plaidml_int_op op, const std::vector<TensorDim>& args) {
    std::vector<plaidml_dim_expr*> raw;
    for (const auto& a : args) raw.push_back(a.as_ptr());
    ptr_ = wrap(ffi::call<plaidml_dim_expr*>(plaidml_dim_expr_op, op, raw.size(), raw.data()));
  }
  TensorDim operator-() const { return TensorDim(PLAIDML_INT_OP_NEG, {*this}); }
  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_dim_expr_repr, as_ptr())); }
  plaidml_dim_expr* as_ptr() const { return ptr_.get(); }

 private:
  static std::shared_ptr<plaidml_dim_expr> wrap(plaidml_dim_expr* p) { return ffi::own(p, plaidml_dim_expr_free); }
  std::shared_ptr<plaidml_dim_expr> ptr_;
};

// ---- TensorIndex: an index variable or an affine polynomial of them -----------
class TensorIndex {
 public:
  explicit TensorIndex(int64_t value) : ptr_(wrap(ffi::call<plaidml_poly_expr*>(plaidml_poly_expr_literal, value))) {}
  explicit TensorIndex(const std::string& name = "")
      : ptr_(wrap(ffi::call<plaidml_poly_expr*>(plaidml_poly_expr_index, name.c_str()))) {}
  TensorIndex(plaidml_int_op op, const std::vector<TensorIndex>& args) {
    std::vector<plaidml_poly_expr*> raw;
    for (const auto& a : args) raw.push_back(a.as_ptr());
    ptr_ = wrap(ffi::call<plaidml_poly_expr*>(plaidml_poly_expr_op, op, raw.size(), raw.data()));
  }
  // index (op) dimension, in either operand order
  TensorIndex(plaidml_int_op op, const TensorIndex& idx, const TensorDim& dim, bool lhs_first) {
    auto dim_poly = wrap(ffi::call<plaidml_poly_expr*>(plaidml_poly_expr_dim, dim.as_ptr()));
    plaidml_poly_expr* raw[2] = {lhs_first ? idx.as_ptr() : dim_poly.get(), lhs_first ? dim_poly.get() : idx.as_ptr()};
    ptr_ = wrap(ffi::call<plaidml_poly_expr*>(plaidml_poly_expr_op, op, static_cast<size_t>(2), raw));
  }
  TensorIndex operator-() const { return TensorIndex(PLAIDML_INT_OP_NEG, {*this}); }
  Constraint operator<(int64_t rhs) const;
  Constraint operator<(const TensorDim& rhs) const;
  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_poly_expr_repr, as_ptr())); }
  plaidml_poly_expr* as_ptr() const { return ptr_.get(); }

 private:
  static std::shared_ptr<plaidml_poly_expr> wrap(plaidml_poly_expr* p) { return ffi::own(p, plaidml_poly_expr_free); }
  std::shared_ptr<plaidml_poly_expr> ptr_;
};

// `lhs < rhs`, which also implies 0 <= lhs
struct Constraint {
  TensorIndex lhs;
  TensorDim rhs;
};
inline Constraint TensorIndex::operator<(int64_t rhs) const { return Constraint{*this, TensorDim(rhs)}; }
inline Constraint TensorIndex::operator<(const TensorDim& rhs) const { return Constraint{*this, rhs}; }

// ---- TensorLens: re-orders dims / idxs between a source and a target layout ---
class TensorLens {
 public:
  TensorLens() = default;
  TensorLens(const std::string& source, const std::string& target) {
    if (source.size() != target.size()) throw ffi_exception("source and target rank mismatch in TensorLens");
    // entry i of the tensor's own order (source) is taken from where its letter sits in the order the
    // caller writes dims and indices in (target)
    for (char c : source) {
      auto pos = target.find(c);
      if (pos == std::string::npos) throw ffi_exception("source and target dims mismatch in TensorLens");
      map_.push_back(pos);
    }
  }
  template <typename T>
  std::vector<T> apply(const std::vector<T>& dims) const {
    if (map_.empty()) return dims;
    if (dims.size() != map_.size()) throw ffi_exception("rank mismatch in TensorLens apply");
    std::vector<T> ret;
    for (size_t m : map_) ret.push_back(dims[m]);
    return ret;
  }

 private:
  std::vector<size_t> map_;
};

// ---- Tensor ----------------------------------------------------------------------
class Tensor {
 public:
  Tensor() = default;
  explicit Tensor(plaidml_expr* ptr) : ptr_(wrap(ptr)) {}
  explicit Tensor(int value) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_int, static_cast<int64_t>(value)))) {}
  explicit Tensor(unsigned value) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_uint, static_cast<uint64_t>(value)))) {}
  explicit Tensor(uint64_t value) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_uint, value))) {}
  explicit Tensor(int64_t value) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_int, value))) {}
  explicit Tensor(double value) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_float, value))) {}
  explicit Tensor(const TensorDim& dim) : ptr_(wrap(ffi::call<plaidml_expr*>(plaidml_expr_dim, dim.as_ptr()))) {}
  Tensor(const Tensor& rhs, const TensorLens& lens) : ptr_(rhs.ptr_), lens_(lens) {}

  // builds an IndexedTensor for use inside a Contraction
  template <typename... Ts>
  IndexedTensor operator()(Ts... idxs) const;
  IndexedTensor operator()(const std::vector<TensorIndex>& idxs) const;

  Tensor operator-() const;
  Tensor operator~() const;
  Tensor operator!() const;

  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_expr_repr, as_ptr())); }
  TensorShape compute_shape() const { return TensorShape(ffi::call<plaidml_shape*>(plaidml_expr_get_shape, as_ptr())); }
  DType dtype() const { return static_cast<DType>(ffi::call<plaidml_datatype>(plaidml_expr_get_dtype, as_ptr())); }
  size_t rank() const { return ffi::call<size_t>(plaidml_expr_get_rank, as_ptr()); }

  // unifies the tensor's sizes with the given dimensions
  void bind_dims(const std::vector<TensorDim>& dims) const {
    std::vector<plaidml_dim_expr*> raw;
    for (const auto& d : lens_.apply(dims)) raw.push_back(d.as_ptr());
    ffi::call_void(plaidml_expr_bind_dims, as_ptr(), raw.size(), raw.data());
  }
  template <typename... Ts>
  void bind_dims(Ts... dims) const {
    bind_dims(std::vector<TensorDim>{dims...});
  }

  Tensor element(size_t ordinal) const { return Tensor(ffi::call<plaidml_expr*>(plaidml_expr_element, as_ptr(), ordinal)); }
  Tensor use(const TensorLens& lens) const { return Tensor(*this, lens); }
  const TensorLens& lens() const { return lens_; }
  plaidml_expr* as_ptr() const { return ptr_.get(); }
  void* raw_ptr() const { return ffi::call<void*>(plaidml_expr_ptr, as_ptr()); }

 private:
  static std::shared_ptr<plaidml_expr> wrap(plaidml_expr* p) { return ffi::own(p, plaidml_expr_free); }
  std::shared_ptr<plaidml_expr> ptr_;
  TensorLens lens_;
};

using TensorVec = std::vector<Tensor>;

// ---- IndexedTensor: T(i, j) and combinations of them ---------------------------
class IndexedTensor {
 public:
  IndexedTensor() = default;
  IndexedTensor(const Tensor& ref, const std::vector<TensorIndex>& idxs) : ref_(ref), idxs_(idxs) {}
  IndexedTensor(plaidml_combo_op op, const std::vector<IndexedTensor>& operands) : op_(op), operands_(operands) {}
  IndexedTensor operator+(const IndexedTensor& rhs) const { return IndexedTensor(PLAIDML_COMBO_OP_ADD, {*this, rhs}); }
  IndexedTensor operator*(const IndexedTensor& rhs) const { return IndexedTensor(PLAIDML_COMBO_OP_MUL, {*this, rhs}); }
  IndexedTensor operator==(const IndexedTensor& rhs) const { return IndexedTensor(PLAIDML_COMBO_OP_EQ, {*this, rhs}); }

 private:
  friend class Contraction;
  plaidml_combo_op op_ = PLAIDML_COMBO_OP_NONE;
  Tensor ref_;
  std::vector<TensorIndex> idxs_;
  std::vector<IndexedTensor> operands_;
};

// (lhs == rhs) ? true_case : 0 inside a contraction
inline IndexedTensor cond(const IndexedTensor& lhs, const IndexedTensor& rhs, const IndexedTensor& true_case) {
  return IndexedTensor(PLAIDML_COMBO_OP_COND, {lhs, rhs, true_case});
}

// ---- Contraction -------------------------------------------------------------------
class Contraction {
 public:
  explicit Contraction(const TensorLens& lens, const std::string& name = "") : name_(name), lens_(lens) {}
  explicit Contraction(const std::string& name = "") : name_(name) {}
  Contraction(const std::vector<TensorDim>& dims, const std::vector<TensorIndex>& idxs, const std::string& name = "")
      : name_(name), outDims_(dims), outIdxs_(idxs) {}

  template <typename... Ts>
  Contraction& outShape(Ts... dims) {
    outDims_ = std::vector<TensorDim>{TensorDim(dims)...};
    return *this;
  }
  Contraction& outShape(const std::vector<TensorDim>& dims) {
    outDims_ = dims;
    return *this;
  }
  Contraction& outShape(const std::vector<int64_t>& dims) {
    outDims_.clear();
    for (int64_t d : dims) outDims_.emplace_back(d);
    return *this;
  }
  template <typename... Ts>
  Contraction& outAccess(Ts... idxs) {
    outIdxs_ = std::vector<TensorIndex>{TensorIndex(idxs)...};
    return *this;
  }
  Contraction& outAccess(const std::vector<TensorIndex>& idxs) {
    outIdxs_ = idxs;
    return *this;
  }
  Contraction& assign(const IndexedTensor& rhs) { return set(PLAIDML_AGG_OP_ASSIGN, rhs); }
  Contraction& max(const IndexedTensor& rhs) { return set(PLAIDML_AGG_OP_MAX, rhs); }
  Contraction& min(const IndexedTensor& rhs) { return set(PLAIDML_AGG_OP_MIN, rhs); }
  Contraction& product(const IndexedTensor& rhs) { return set(PLAIDML_AGG_OP_PROD, rhs); }
  Contraction& sum(const IndexedTensor& rhs) { return set(PLAIDML_AGG_OP_SUM, rhs); }
  Contraction& init(const Tensor& rhs) {
    init_ = rhs;
    return *this;
  }
  Contraction& add_constraint(const Constraint& constraint) {
    constraints_.push_back(constraint);
    return *this;
  }
  Contraction& add_constraints(const std::vector<Constraint>& constraints) {
    constraints_.insert(constraints_.end(), constraints.begin(), constraints.end());
    return *this;
  }

  Tensor build() {
    if (rhs_.op_ == PLAIDML_COMBO_OP_NONE && !rhs_.ref_.as_ptr()) throw ffi_exception("contraction without an aggregated expression");
    std::vector<plaidml_poly_expr*> idxs;
    for (const auto& i : lens_.apply(outIdxs_)) idxs.push_back(i.as_ptr());
    std::vector<plaidml_dim_expr*> dims;
    for (const auto& d : lens_.apply(outDims_)) dims.push_back(d.as_ptr());
    if (idxs.size() != dims.size()) throw ffi_exception("outShape and outAccess must have the same rank");
    Tensor result(ffi::call<plaidml_expr*>(plaidml_expr_contraction, agg_, rhs_.op_, idxs.size(), idxs.data(), dims.data(),
                                           init_.as_ptr(), name_.c_str()));
    std::vector<IndexedTensor> operands = rhs_.op_ == PLAIDML_COMBO_OP_NONE ? std::vector<IndexedTensor>{rhs_} : rhs_.operands_;
    for (const IndexedTensor& operand : operands) {
      if (operand.op_ != PLAIDML_COMBO_OP_NONE) throw ffi_exception("nested combinations are not valid inside a contraction");
      std::vector<plaidml_poly_expr*> raw;
      for (const auto& i : operand.ref_.lens().apply(operand.idxs_)) raw.push_back(i.as_ptr());
      ffi::call_void(plaidml_contraction_add_operand, result.as_ptr(), operand.ref_.as_ptr(), raw.size(), raw.data());
    }
    for (const Constraint& c : constraints_)
      ffi::call_void(plaidml_contraction_add_constraint, result.as_ptr(), c.lhs.as_ptr(), c.rhs.as_ptr());
    ffi::call_void(plaidml_contraction_build, result.as_ptr());
    return result;
  }
  operator Tensor() { return build(); }  // NOLINT: the reference converts implicitly

 private:
  Contraction& set(plaidml_agg_op agg, const IndexedTensor& rhs) {
    agg_ = agg;
    rhs_ = rhs;
    return *this;
  }
  std::string name_;
  TensorLens lens_;
  std::vector<TensorDim> outDims_;
  std::vector<TensorIndex> outIdxs_;
  plaidml_agg_op agg_ = PLAIDML_AGG_OP_NONE;
  IndexedTensor rhs_;
  std::vector<Constraint> constraints_;
  Tensor init_;
};

template <typename... Ts>
inline IndexedTensor Tensor::operator()(Ts... idxs) const {
  return IndexedTensor(*this, std::vector<TensorIndex>{TensorIndex(idxs)...});
}
inline IndexedTensor Tensor::operator()(const std::vector<TensorIndex>& idxs) const { return IndexedTensor(*this, idxs); }

// ---- program inputs and constants ----------------------------------------------
inline Tensor Constant(const Buffer& buffer, const std::string& name = "") {
  return Tensor(ffi::call<plaidml_expr*>(plaidml_expr_constant, buffer.as_ptr(), name.c_str()));
}
inline Tensor Constant(int value) { return Tensor(value); }
inline Tensor Constant(int64_t value) { return Tensor(value); }
inline Tensor Constant(uint64_t value) { return Tensor(value); }
inline Tensor Constant(double value) { return Tensor(value); }

inline Tensor Placeholder(const TensorShape& shape, const std::string& name = "") {
  return Tensor(ffi::call<plaidml_expr*>(plaidml_expr_input, shape.as_ptr(), name.c_str()));
}
inline Tensor Placeholder(DType dtype, const std::vector<int64_t>& dims, const std::string& name = "") {
  return Placeholder(TensorShape(dtype, dims), name);
}
inline Tensor Zero() { return Tensor(0); }

// ---- intrinsics ----------------------------------------------------------------------
inline Tensor intrinsicCall(const std::string& fn, const TensorVec& args, const std::string& name = "") {
  std::vector<plaidml_expr*> raw;
  for (const auto& a : args) raw.push_back(a.as_ptr());
  return Tensor(ffi::call<plaidml_expr*>(plaidml_expr_intrinsic, fn.c_str(), raw.size(), raw.data(), name.c_str()));
}

namespace details {
inline Tensor as_tensor(const Tensor& t) { return t; }
inline Tensor as_tensor(int v) { return Tensor(v); }
inline Tensor as_tensor(unsigned v) { return Tensor(v); }
inline Tensor as_tensor(int64_t v) { return Tensor(v); }
inline Tensor as_tensor(uint64_t v) { return Tensor(v); }
inline Tensor as_tensor(double v) { return Tensor(v); }
inline Tensor as_tensor(const TensorDim& d) { return Tensor(d); }
}  // namespace details

template <typename... Ts>
Tensor intrinsic(const std::string& fn, Ts... args) {
  return intrinsicCall(fn, TensorVec{details::as_tensor(args)...});
}

inline Tensor cast(const Tensor& x, DType dtype) {
  return Tensor(ffi::call<plaidml_expr*>(plaidml_expr_cast, x.as_ptr(), static_cast<plaidml_datatype>(dtype)));
}
inline Tensor select(const Tensor& cond, const Tensor& true_case, const Tensor& false_case) {
  return intrinsicCall("select", {cond, true_case, false_case});
}
inline Tensor ceil(const Tensor& x) { return intrinsicCall("ceil", {x}); }
inline Tensor exp(const Tensor& x) { return intrinsicCall("exp", {x}); }
inline Tensor floor(const Tensor& x) { return intrinsicCall("floor", {x}); }
inline Tensor ident(const Tensor& x) { return intrinsicCall("ident", {x}); }
inline Tensor log(const Tensor& x) { return intrinsicCall("log", {x}); }
inline Tensor relu(const Tensor& x, const std::string& name = "") { return intrinsicCall("relu", {x}, name); }
inline Tensor round(const Tensor& x) { return intrinsicCall("round", {x}); }
inline Tensor sqrt(const Tensor& x) { return intrinsicCall("sqrt", {x}); }
inline Tensor tanh(const Tensor& x) { return intrinsicCall("tanh", {x}); }
inline Tensor shape(const Tensor& x) { return intrinsicCall("shape", {x}); }
inline Tensor sin(const Tensor& x) { return intrinsicCall("sin", {x}); }
inline Tensor cos(const Tensor& x) { return intrinsicCall("cos", {x}); }
inline Tensor tan(const Tensor& x) { return intrinsicCall("tan", {x}); }
inline Tensor sinh(const Tensor& x) { return intrinsicCall("sinh", {x}); }
inline Tensor cosh(const Tensor& x) { return intrinsicCall("cosh", {x}); }
inline Tensor asin(const Tensor& x) { return intrinsicCall("asin", {x}); }
inline Tensor acos(const Tensor& x) { return intrinsicCall("acos", {x}); }
inline Tensor atan(const Tensor& x) { return intrinsicCall("atan", {x}); }
inline Tensor asinh(const Tensor& x) { return intrinsicCall("asinh", {x}); }
inline Tensor acosh(const Tensor& x) { return intrinsicCall("acosh", {x}); }
inline Tensor atanh(const Tensor& x) { return intrinsicCall("atanh", {x}); }
inline Tensor erf(const Tensor& x) { return intrinsicCall("erf", {x}); }
inline Tensor pow(const Tensor& x, const Tensor& y) { return intrinsicCall("pow", {x, y}); }
// a tensor of shape `dims` whose elements are their own coordinate along `axis`
inline Tensor index(const std::vector<TensorDim>& dims, size_t axis) {
  TensorVec args = {Tensor(static_cast<int64_t>(axis))};
  for (const auto& d : dims) args.emplace_back(d);
  return intrinsicCall("index", args);
}
inline Tensor reshape(const Tensor& x, const std::vector<int64_t>& dims) {
  TensorVec args = {x};
  for (int64_t d : dims) args.emplace_back(d);
  return intrinsicCall("reshape", args);
}
inline Tensor reshape(const Tensor& x, const std::vector<TensorDim>& dims) {
  TensorVec args = {x};
  for (const auto& d : dims) args.emplace_back(d);
  return intrinsicCall("reshape", args);
}

inline Tensor Tensor::operator-() const { return intrinsicCall("neg", {*this}); }
inline Tensor Tensor::operator~() const { return intrinsicCall("bit_not", {*this}); }
inline Tensor Tensor::operator!() const { return intrinsicCall("logical_not", {*this}); }

// ---- operators -------------------------------------------------------------------------
#define PLAIDML_EDSL_IDX_DIM_OPS(_op_, _int_op_, _fn_)                                                                  \
  inline TensorIndex operator _op_(const TensorIndex& l, const TensorIndex& r) { return TensorIndex(_int_op_, {l, r}); } \
  inline TensorIndex operator _op_(const TensorIndex& l, int64_t r) { return TensorIndex(_int_op_, {l, TensorIndex(r)}); } \
  inline TensorIndex operator _op_(int64_t l, const TensorIndex& r) { return TensorIndex(_int_op_, {TensorIndex(l), r}); } \
  inline TensorIndex operator _op_(const TensorIndex& l, const TensorDim& r) { return TensorIndex(_int_op_, l, r, true); } \
  inline TensorIndex operator _op_(const TensorDim& l, const TensorIndex& r) { return TensorIndex(_int_op_, r, l, false); } \
  inline Tensor operator _op_(const Tensor& l, const TensorDim& r) { return intrinsic(_fn_, l, Tensor(r)); }            \
  inline Tensor operator _op_(const TensorDim& l, const Tensor& r) { return intrinsic(_fn_, Tensor(l), r); }            \
  inline TensorDim operator _op_(const TensorDim& l, const TensorDim& r) { return TensorDim(_int_op_, {l, r}); }        \
  inline TensorDim operator _op_(int64_t l, const TensorDim& r) { return TensorDim(_int_op_, {TensorDim(l), r}); }      \
  inline TensorDim operator _op_(const TensorDim& l, int64_t r) { return TensorDim(_int_op_, {l, TensorDim(r)}); }

PLAIDML_EDSL_IDX_DIM_OPS(+, PLAIDML_INT_OP_ADD, "add")
PLAIDML_EDSL_IDX_DIM_OPS(-, PLAIDML_INT_OP_SUB, "sub")
PLAIDML_EDSL_IDX_DIM_OPS(*, PLAIDML_INT_OP_MUL, "mul")
PLAIDML_EDSL_IDX_DIM_OPS(/, PLAIDML_INT_OP_DIV, "div")
#undef PLAIDML_EDSL_IDX_DIM_OPS

inline TensorDim max(const TensorDim& l, const TensorDim& r) { return TensorDim(PLAIDML_INT_OP_MAX, {l, r}); }
inline TensorDim max(int64_t l, const TensorDim& r) { return TensorDim(PLAIDML_INT_OP_MAX, {TensorDim(l), r}); }
inline TensorDim max(const TensorDim& l, int64_t r) { return TensorDim(PLAIDML_INT_OP_MAX, {l, TensorDim(r)}); }
inline TensorDim min(const TensorDim& l, const TensorDim& r) { return TensorDim(PLAIDML_INT_OP_MIN, {l, r}); }
inline TensorDim min(int64_t l, const TensorDim& r) { return TensorDim(PLAIDML_INT_OP_MIN, {TensorDim(l), r}); }
inline TensorDim min(const TensorDim& l, int64_t r) { return TensorDim(PLAIDML_INT_OP_MIN, {l, TensorDim(r)}); }

#define PLAIDML_EDSL_TENSOR_OPS(_op_, _fn_)                                                     \
  inline Tensor operator _op_(const Tensor& l, const Tensor& r) { return intrinsic(_fn_, l, r); } \
  inline Tensor operator _op_(const Tensor& l, int r) { return intrinsic(_fn_, l, r); }           \
  inline Tensor operator _op_(const Tensor& l, int64_t r) { return intrinsic(_fn_, l, r); }       \
  inline Tensor operator _op_(const Tensor& l, uint64_t r) { return intrinsic(_fn_, l, r); }      \
  inline Tensor operator _op_(const Tensor& l, double r) { return intrinsic(_fn_, l, r); }        \
  inline Tensor operator _op_(int l, const Tensor& r) { return intrinsic(_fn_, l, r); }           \
  inline Tensor operator _op_(int64_t l, const Tensor& r) { return intrinsic(_fn_, l, r); }       \
  inline Tensor operator _op_(uint64_t l, const Tensor& r) { return intrinsic(_fn_, l, r); }      \
  inline Tensor operator _op_(double l, const Tensor& r) { return intrinsic(_fn_, l, r); }

PLAIDML_EDSL_TENSOR_OPS(+, "add")
PLAIDML_EDSL_TENSOR_OPS(-, "sub")
PLAIDML_EDSL_TENSOR_OPS(*, "mul")
PLAIDML_EDSL_TENSOR_OPS(/, "div")
PLAIDML_EDSL_TENSOR_OPS(==, "cmp_eq")
PLAIDML_EDSL_TENSOR_OPS(!=, "cmp_ne")
PLAIDML_EDSL_TENSOR_OPS(<, "cmp_lt")
PLAIDML_EDSL_TENSOR_OPS(>, "cmp_gt")
PLAIDML_EDSL_TENSOR_OPS(<=, "cmp_le")
PLAIDML_EDSL_TENSOR_OPS(>=, "cmp_ge")
PLAIDML_EDSL_TENSOR_OPS(%, "mod")
PLAIDML_EDSL_TENSOR_OPS(<<, "bit_shl")
PLAIDML_EDSL_TENSOR_OPS(>>, "bit_shr")
PLAIDML_EDSL_TENSOR_OPS(&, "bit_and")
PLAIDML_EDSL_TENSOR_OPS(|, "bit_or")
PLAIDML_EDSL_TENSOR_OPS(^, "bit_xor")
PLAIDML_EDSL_TENSOR_OPS(&&, "logical_and")
PLAIDML_EDSL_TENSOR_OPS(||, "logical_or")
#undef PLAIDML_EDSL_TENSOR_OPS

inline Tensor abs(const Tensor& x) { return select(x < 0.0, -x, x); }

// ---- special operations: argsort, gather, scatter (plaidml/edsl/edsl.h:800-811, 1034-1066, 1625-1765) ----
enum class SortDirection : uint64_t { ASC, DESC };

inline Tensor argsort(const Tensor& x, int axis = -1, SortDirection direction = SortDirection::ASC) {
  return intrinsicCall("argsort", {x, Tensor(static_cast<int64_t>(axis)), Tensor(static_cast<int64_t>(direction))});
}

enum class InterpolationMode : uint64_t { NEAREST, LINEAR, CUBIC, NONE };
enum class NearestMode : uint64_t { ROUND_PREFER_FLOOR, ROUND_PREFER_CEIL, FLOOR, CEIL, SIMPLE, NONE };
enum class GatherMode : uint64_t { NORMAL, ND };
enum class OutOfBoundsMode : uint64_t { GATHER_EDGE_PADDED_INPUT, RETURN_ZERO };
enum class ScatterMode : uint64_t { NORMAL, UPDATE_SLICE, UPDATE_ELT, UPDATE_ND };

// dims values in [0, 1) drawn from the three-word state, and the state advanced past them
// (plaidml/edsl/edsl.h:971-979, pmlc/rt/prng.cc)
inline std::pair<Tensor, Tensor> prng(const Tensor& state, const std::vector<int64_t>& dims) {
  TensorVec args = {state};
  for (int64_t d : dims) args.emplace_back(TensorDim(d));
  Tensor R = intrinsicCall("prng", args);
  return std::make_pair(R.element(0), R.element(1));
}

// the nine-argument gather intrinsic; `gather` below and op::gatherND fill it in
class gatherBuilder {
 public:
  gatherBuilder(Tensor x, Tensor y, uint64_t axis, InterpolationMode interpolation_mode, NearestMode nearest_mode,
                OutOfBoundsMode out_of_bounds_mode, float cube_coeff)
      : x_(x), y_(y), axis_(axis), cube_coeff_(cube_coeff), mode_(GatherMode::NORMAL), out_of_bounds_mode_(out_of_bounds_mode),
        nearest_mode_(nearest_mode), interpolation_mode_(interpolation_mode) {}
  gatherBuilder(Tensor x, Tensor y, uint64_t batch_dims, InterpolationMode interpolation_mode)
      : x_(x), y_(y), batch_dims_(batch_dims), mode_(GatherMode::ND), interpolation_mode_(interpolation_mode) {}
  Tensor build() const {
    return intrinsicCall("gather", {x_, y_, Tensor(axis_), Tensor(static_cast<uint64_t>(interpolation_mode_)),
                                    Tensor(static_cast<uint64_t>(nearest_mode_)), Tensor(static_cast<double>(cube_coeff_)),
                                    Tensor(static_cast<uint64_t>(mode_)), Tensor(batch_dims_),
                                    Tensor(static_cast<uint64_t>(out_of_bounds_mode_))});
  }

 private:
  Tensor x_, y_;
  uint64_t axis_ = 0, batch_dims_ = 0;
  float cube_coeff_ = -0.75;
  GatherMode mode_ = GatherMode::NORMAL;
  OutOfBoundsMode out_of_bounds_mode_ = OutOfBoundsMode::GATHER_EDGE_PADDED_INPUT;
  NearestMode nearest_mode_ = NearestMode::ROUND_PREFER_FLOOR;
  InterpolationMode interpolation_mode_ = InterpolationMode::NONE;
};

// x taken along `axis` at the positions y; a number in place of y reads that one position
class gather {
 public:
  gather(const Tensor& x, const Tensor& y) : x_(x), y_(y) {}
  gather(const Tensor& x, int i) : x_(x), y_(cast(index({TensorDim(1)}, 0), DType::INT32) + i) {}
  gather(const Tensor& x, int64_t i) : x_(x), y_(cast(index({TensorDim(1)}, 0), DType::INT64) + i) {}
  gather(const Tensor& x, uint64_t i) : x_(x), y_(cast(index({TensorDim(1)}, 0), DType::UINT64) + i) {}
  gather(const Tensor& x, float f) : x_(x), y_(cast(index({TensorDim(1)}, 0), DType::FLOAT32) + static_cast<double>(f)) {}
  gather(const Tensor& x, double f) : x_(x), y_(cast(index({TensorDim(1)}, 0), DType::FLOAT64) + f) {}
  gather& axis(int64_t axis) {
    if (axis < 0) axis += static_cast<int64_t>(x_.rank());
    axis_ = static_cast<uint64_t>(axis);
    return *this;
  }
  gather& interpolationMode(InterpolationMode mode) { interpolation_mode_ = mode; return *this; }
  gather& nearestMode(NearestMode mode) { nearest_mode_ = mode; return *this; }
  gather& cubeCoeff(float cube_coeff) { cube_coeff_ = cube_coeff; return *this; }
  gather& outOfBoundsMode(OutOfBoundsMode mode) { out_of_bounds_mode_ = mode; return *this; }
  operator Tensor() const {  // NOLINT: the reference converts implicitly
    return gatherBuilder(x_, y_, axis_, interpolation_mode_, nearest_mode_, out_of_bounds_mode_, cube_coeff_).build();
  }

 private:
  Tensor x_, y_;
  uint64_t axis_ = 0;
  InterpolationMode interpolation_mode_ = InterpolationMode::NONE;
  NearestMode nearest_mode_ = NearestMode::ROUND_PREFER_FLOOR;
  OutOfBoundsMode out_of_bounds_mode_ = OutOfBoundsMode::GATHER_EDGE_PADDED_INPUT;
  float cube_coeff_ = -0.75;
};

// a copy of x with the elements of z written (or, in NORMAL mode, added) at the places y names
class scatter {
 public:
  scatter(const Tensor& x, const Tensor& y, const Tensor& z) : x_(x), y_(y), z_(z) {}
  scatter& axis(int64_t axis) {
    if (axis < 0) axis += static_cast<int64_t>(x_.rank());
    axis_ = axis;
    return *this;
  }
  scatter& mode(ScatterMode mode) { mode_ = mode; return *this; }
  Tensor build() const { return intrinsicCall("scatter", {x_, y_, z_, Tensor(axis_), Tensor(static_cast<uint64_t>(mode_))}); }
  operator Tensor() const { return build(); }  // NOLINT

 private:
  Tensor x_, y_, z_;
  int64_t axis_ = 0;
  ScatterMode mode_ = ScatterMode::NORMAL;
};

// ---- Value: the variant handed to the operation library --------------------------
class Value {
 public:
  Value() : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_none))) {}
  explicit Value(plaidml_value* ptr) : ptr_(wrap(ptr)) {}
  explicit Value(int8_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(int16_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(int32_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(int64_t v) : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_int, v))) {}
  explicit Value(uint8_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(uint16_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(uint32_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(uint64_t v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(bool v) : Value(static_cast<int64_t>(v)) {}
  explicit Value(double v) : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_float, v))) {}
  explicit Value(const std::string& v) : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_str, v.c_str()))) {}
  explicit Value(const char* v) : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_str, v))) {}
  explicit Value(const TensorDim& dim) : ptr_(wrap(ffi::call<plaidml_value*>(plaidml_value_dim, dim.as_ptr()))) {}
  explicit Value(const Tensor& tensor) {
    ptr_ = tensor.as_ptr() ? wrap(ffi::call<plaidml_value*>(plaidml_value_expr, tensor.as_ptr()))
                           : wrap(ffi::call<plaidml_value*>(plaidml_value_none));
  }
  explicit Value(const std::vector<Value>& tuple) {
    std::vector<plaidml_value*> raw;
    for (const auto& v : tuple) raw.push_back(v.as_ptr());
    ptr_ = wrap(ffi::call<plaidml_value*>(plaidml_value_tuple, raw.size(), raw.data()));
  }

  std::string str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_value_repr, as_ptr())); }
  plaidml_value_kind kind() const { return ffi::call<plaidml_value_kind>(plaidml_value_get_kind, as_ptr()); }
  bool is_none() const { return kind() == PLAIDML_VALUE_NONE; }
  bool is_int() const { return kind() == PLAIDML_VALUE_INT; }
  bool is_float() const { return kind() == PLAIDML_VALUE_FLOAT; }
  bool is_tensor() const { return kind() == PLAIDML_VALUE_EXPR; }
  bool is_tuple() const { return kind() == PLAIDML_VALUE_TUPLE; }
  bool is_str() const { return kind() == PLAIDML_VALUE_STR; }
  bool is_dim() const { return kind() == PLAIDML_VALUE_DIM; }

  bool as_bool() const { return as_int() != 0; }
  int64_t as_int() const { return ffi::call<int64_t>(plaidml_value_int_get, as_ptr()); }
  double as_float() const { return ffi::call<double>(plaidml_value_float_get, as_ptr()); }
  std::string as_str() const { return ffi::str(ffi::call<plaidml_string*>(plaidml_value_str_get, as_ptr())); }
  // numbers and dims convert to scalar tensors
  Tensor as_tensor() const {
    if (is_tensor()) return Tensor(ffi::call<plaidml_expr*>(plaidml_value_expr_get, as_ptr()));
    if (is_dim()) return Tensor(as_dim());
    if (is_float()) return Tensor(as_float());
    if (is_int()) return Tensor(as_int());
    throw ffi_exception("Value cannot be converted to a Tensor");
  }
  TensorDim as_dim() const {
    return TensorDim(ffi::own(ffi::call<plaidml_dim_expr*>(plaidml_value_dim_get, as_ptr()), plaidml_dim_expr_free));
  }
  std::vector<Value> as_tuple() const {
    auto tuple = ffi::own(ffi::call<plaidml_tuple*>(plaidml_value_tuple_get, as_ptr()), plaidml_tuple_free);
    std::vector<Value> ret;
    for (size_t i = 0; i < tuple->size; ++i) ret.emplace_back(tuple->elts[i]);
    return ret;
  }
  std::vector<int64_t> as_int_tuple() const {
    std::vector<int64_t> ret;
    for (const auto& v : as_tuple()) ret.push_back(v.as_int());
    return ret;
  }
  std::vector<int64_t> as_int_tuple_or_empty() const { return is_none() ? std::vector<int64_t>{} : as_int_tuple(); }
  plaidml_value* as_ptr() const { return ptr_.get(); }

 private:
  static std::shared_ptr<plaidml_value> wrap(plaidml_value* p) { return ffi::own(p, plaidml_value_free); }
  std::shared_ptr<plaidml_value> ptr_;
};

inline Value None() { return Value(); }

namespace details {
inline Value as_value(const Value& v) { return v; }
inline Value as_value(const Tensor& t) { return Value(t); }
inline Value as_value(const TensorDim& d) { return Value(d); }
inline Value as_value(const std::string& s) { return Value(s); }
inline Value as_value(const char* s) { return Value(s); }
inline Value as_value(bool v) { return Value(v); }
inline Value as_value(int v) { return Value(static_cast<int64_t>(v)); }
inline Value as_value(int64_t v) { return Value(v); }
inline Value as_value(uint64_t v) { return Value(v); }
inline Value as_value(double v) { return Value(v); }
// a vector among the elements becomes a nested tuple
template <typename T>
Value as_value(const std::vector<T>& v) {
  std::vector<Value> vec;
  for (const auto& e : v) vec.push_back(as_value(e));
  return Value(vec);
}
}  // namespace details

template <typename... Ts>
Value make_tuple(Ts... elts) {
  return Value(std::vector<Value>{details::as_value(elts)...});
}
template <typename T>
Value make_tuple(const std::vector<T>& elts) {
  std::vector<Value> vec;
  for (const auto& e : elts) vec.push_back(details::as_value(e));
  return Value(vec);
}
inline Value make_tuple(const std::vector<Value>& elts) { return Value(elts); }

// ---- program construction ------------------------------------------------------------
inline Program buildProgram(const std::string& name, const TensorVec& inputs, const TensorVec& outputs) {
  std::vector<plaidml_expr*> in, out;
  for (const auto& t : inputs) in.push_back(t.as_ptr());
  for (const auto& t : outputs) out.push_back(t.as_ptr());
  return Program(ffi::call<plaidml_program*>(plaidml_build, name.c_str(), in.size(), in.data(),
                                             static_cast<plaidml_shape**>(nullptr), out.size(), out.data()));
}

inline std::ostream& operator<<(std::ostream& os, const Tensor& x) { return os << x.str(); }
inline std::ostream& operator<<(std::ostream& os, const TensorDim& x) { return os << x.str(); }
inline std::ostream& operator<<(std::ostream& os, const TensorIndex& x) { return os << x.str(); }
inline std::ostream& operator<<(std::ostream& os, const Value& x) { return os << x.str(); }

using Dictionary = std::unordered_map<std::string, Value>;

// Layers group operations for readers of the program text; this backend inlines them.  The operand list is
// not checked: a body that reads a tensor missing from it builds here, where the reference rejects the
// program (plaidml/edsl/tests/edsl_test.cc:2200-2205).
inline Tensor layer(const std::string&, const TensorVec&, const Dictionary&, const std::function<Tensor()>& fn) { return fn(); }
inline Tensor layer(const std::string&, const TensorVec&, const std::function<Tensor()>& fn) { return fn(); }
inline TensorVec layer(const std::string&, const TensorVec&, const Dictionary&, const std::function<TensorVec()>& fn) { return fn(); }
// A trace marker passes its tensor through.
inline Tensor trace(const Tensor& x, const std::string&) { return x; }

}  // namespace edsl
}  // namespace plaidml

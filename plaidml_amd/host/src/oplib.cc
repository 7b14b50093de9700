// The operation library behind plaidml_op_make: the subset of the reference's
// plaidml/op/lib/ops.cc that the contraction hot path uses, written (as there) on top
// of the EDSL itself, so that every operation becomes Tile contractions and
// elementwise operations.
//
//   convolution  ops.cc:879-1467 (forward mode; NXC / NCX inputs, XCK / KCX filters;
//                group layouts NONE and IN_C; autogroup UNGROUPED / EXPLICIT / DEPTHWISE)
//   padding rule ops.cc:347-382
//   pool         ops.cc:2562-2703        dot      ops.cc:1512-1561
//   argmax       ops.cc:505-521          clip     ops.cc:584-606
//   max / min / sum / mean via AggregationAxes ops.cc:71-127,1970-2003,3424-
//   maximum / minimum ops.cc:1958-1968   relu     ops.cc:2705-2728
//   softmax      ops.cc:3049-3098 (softmax over the last axis)
//   data movement and simple arithmetic (every one a single contraction or elementwise chain):
//   abs 439-447, concatenate 608-668, cumsum 1490-1510, elu 1563-1584, explicit_padding 1586-1685
//   (CONSTANT and EDGE), flip 1687-1725, hard_sigmoid 1803-1820, prod 2532-, repeat 2782-2819,
//   reshape 2821-2885, sigmoid 2906-2915, spatial_padding 3129- (NXC and NCX), square 3380-3384,
//   squeeze 3386-3422, tile 3454-3489, transpose 3491-3537, unsqueeze 3539-3584, variance 3586-3632
#include <functional>
#include <map>
#include <set>

#include "ffi_internal.h"
#include "plaidml/op/op.h"

using namespace plaidml;        // NOLINT
using namespace plaidml::edsl;  // NOLINT
using plaidml::op::AutoGroupMode;
using plaidml::op::AutoPadMode;
using plaidml::op::ConvDerivMode;
using plaidml::op::EpsMode;
using plaidml::op::GroupLayout;
using plaidml::op::PoolMode;
using plaidml::op::TensorLayout;

namespace {

template <typename E>
E validate(int64_t raw) {
  if (raw < 0 || raw >= static_cast<int64_t>(E::_LAST)) throw std::runtime_error("Invalid enumeration value in operation arguments");
  return static_cast<E>(raw);
}

std::pair<TensorDim, TensorDim> compute_padding_and_output_size(const TensorDim& input_size, const TensorDim& filter_size,
                                                                int64_t stride, AutoPadMode mode, int64_t pad_lo,
                                                                int64_t pad_hi, int64_t dilation, int64_t data_dilation,
                                                                bool use_ceil) {
  TensorDim i_eff = (data_dilation * (input_size - 1)) + 1;
  TensorDim f_eff = (dilation * (filter_size - 1)) + 1;
  const int64_t ceil_term = use_ceil ? stride - 1 : 0;
  switch (mode) {
    case AutoPadMode::EXPLICIT:
      return {TensorDim(pad_lo), (i_eff + pad_lo + pad_hi - f_eff + stride + ceil_term) / stride};
    case AutoPadMode::VALID:
      return {TensorDim(0), (i_eff - f_eff + stride + ceil_term) / stride};
    case AutoPadMode::SAME_LOWER:
    case AutoPadMode::SAME_UPPER: {
      TensorDim out = (i_eff + stride - 1) / stride;
      const int64_t lower = mode == AutoPadMode::SAME_LOWER ? 1 : 0;
      TensorDim pad = (edsl::max(0, (out - 1) * stride + f_eff - i_eff) + lower) / 2;
      return {pad, out};
    }
    default:
      throw std::runtime_error("Unexpected autopadding mode");
  }
}

struct AggregationAxes {
  std::vector<TensorIndex> src_idxs, dst_idxs, reduce_idxs;
  std::vector<TensorDim> src_dims, dst_dims, reduce_dims;
  std::set<size_t> axes;

  AggregationAxes(size_t ndims, const Value& in_axes, bool keepdims) : src_idxs(ndims), src_dims(ndims) {
    auto norm = [&](int64_t a) {
      if (a < 0) a += static_cast<int64_t>(ndims);
      if (a < 0 || a >= static_cast<int64_t>(ndims)) throw std::out_of_range("axis out of range: " + std::to_string(a));
      return static_cast<size_t>(a);
    };
    if (in_axes.is_none()) {
      for (size_t i = 0; i < ndims; ++i) axes.insert(i);
    } else if (in_axes.is_tuple()) {
      for (const auto& a : in_axes.as_tuple()) axes.insert(norm(a.as_int()));
    } else if (in_axes.is_int()) {
      axes.insert(norm(in_axes.as_int()));
    } else {
      throw std::runtime_error("Invalid Value type for AggregationAxes: in_axes");
    }
    for (size_t a : axes) {
      reduce_idxs.push_back(src_idxs[a]);
      reduce_dims.push_back(src_dims[a]);
    }
    if (keepdims) {
      dst_idxs = src_idxs;
      dst_dims = src_dims;
      for (size_t a : axes) {
        dst_idxs[a] = TensorIndex();
        dst_dims[a] = TensorDim(1);
      }
    } else {
      for (size_t i = 0; i < ndims; ++i) {
        if (!axes.count(i)) {
          dst_idxs.push_back(src_idxs[i]);
          dst_dims.push_back(src_dims[i]);
        }
      }
    }
  }
};

Value reduce(const Value& value, const char* what, plaidml_agg_op agg) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error(std::string(what) + " expects 3 arguments");
  auto I = args[0].as_tensor();
  if (I.rank() == 0) return Value{I};
  auto axes = args[1];
  if (axes.is_tuple() && axes.as_tuple().empty()) return Value{I};
  AggregationAxes ag(I.rank(), axes, args[2].as_bool());
  I.bind_dims(ag.src_dims);
  Contraction c(ag.dst_dims, ag.dst_idxs, what);
  switch (agg) {
    case PLAIDML_AGG_OP_MAX: c.max(I(ag.src_idxs)); break;
    case PLAIDML_AGG_OP_MIN: c.min(I(ag.src_idxs)); break;
    default: c.sum(I(ag.src_idxs)); break;
  }
  Tensor O = c;
  if (std::string(what) == "mean") {
    Tensor denom(1);
    for (size_t a : ag.axes) denom = denom * ag.src_dims.at(a);
    return Value{O / denom};
  }
  return Value{O};
}

Value op_argmax(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("argmax expects 2 arguments");
  auto I = args[0].as_tensor();
  AggregationAxes ag(I.rank(), args[1], false);
  I.bind_dims(ag.src_dims);
  Tensor M = Contraction(ag.dst_dims, ag.dst_idxs, "argmax").max(I(ag.src_idxs));
  Tensor IX = index(ag.reduce_dims, 0);
  Tensor AM = Contraction(ag.dst_dims, ag.dst_idxs, "argmax").max(cond(I(ag.src_idxs), M(ag.dst_idxs), IX(ag.reduce_idxs)));
  return Value{cast(AM, DType::UINT32)};
}

Value op_clip(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("clip expects 3 arguments");
  auto O = args[0].as_tensor();
  if (!args[1].is_none()) {
    auto lo = args[1].as_tensor();
    O = select(O > lo, O, cast(lo, O.dtype()));
  }
  if (!args[2].is_none()) {
    auto hi = args[2].as_tensor();
    O = select(O < hi, O, cast(hi, O.dtype()));
  }
  return Value{O};
}

// ---- convolution (plaidml/op/lib/ops.cc:671-877 validation, :879-1467 construction) ------------------------
// One contraction relates I (data), F (filters) and O (result of the forward pass):
//   O[n, x.., g*(CO/G)+co] += I[n, (s*x + d*k - pad)/dd .., g*(CI/G)+ci] * F[k.., f_ci, f_co]
// deriv_mode picks which of the three is computed from the other two: NONE -> O, DATA -> I (a transposed
// convolution), FILTER -> F.  The group layout says which filter channel dimension carries the group.

size_t nonspatial_dims(TensorLayout layout) {
  switch (layout) {
    case TensorLayout::GKCX:
    case TensorLayout::XGCK: return 3;
    default: return 2;
  }
}

// smallest input extent that yields `output_size` (ops.cc:383-418).  For the SAME modes the reference hands
// back the output extent itself as the input extent; kept, since result shapes must agree with it.
std::pair<TensorDim, TensorDim> compute_padding_and_input_size(const TensorDim& output_size, const TensorDim& filter_size,
                                                               int64_t stride, AutoPadMode mode, int64_t pad_lo, int64_t pad_hi,
                                                               int64_t dilation, int64_t data_dilation) {
  if (data_dilation != 1) throw std::runtime_error("Cannot infer input data size for transposed convolution with data dilation");
  TensorDim f_eff = (dilation * (filter_size - 1)) + 1;
  switch (mode) {
    case AutoPadMode::EXPLICIT: return {TensorDim(pad_lo), output_size * stride - pad_lo - pad_hi + f_eff - stride};
    case AutoPadMode::VALID: return {TensorDim(0), output_size * stride + f_eff - stride};
    case AutoPadMode::SAME_LOWER:
    case AutoPadMode::SAME_UPPER: {
      TensorDim input_size = output_size * stride - stride + 1;
      const int64_t lower = mode == AutoPadMode::SAME_LOWER ? 1 : 0;
      TensorDim pad_before = (edsl::max(0, (output_size - 1) * stride + f_eff - input_size) + lower) / 2;
      return {pad_before, output_size};
    }
    default: throw std::runtime_error("Unexpected autopadding mode");
  }
}

template <typename T>
std::vector<T> data_order(TensorLayout layout, const T& n, const T& c, const std::vector<T>& spatial) {
  std::vector<T> r = {n};
  if (layout == TensorLayout::NCX) r.push_back(c);
  r.insert(r.end(), spatial.begin(), spatial.end());
  if (layout == TensorLayout::NXC) r.push_back(c);
  return r;
}

template <typename T>
std::vector<T> filter_order(TensorLayout layout, const T& g, const T& k, const T& c, const std::vector<T>& spatial) {
  std::vector<T> r;
  if (layout == TensorLayout::GKCX || layout == TensorLayout::KCX) {
    if (layout == TensorLayout::GKCX) r.push_back(g);
    r.push_back(k);
    r.push_back(c);
    r.insert(r.end(), spatial.begin(), spatial.end());
  } else {
    r.insert(r.end(), spatial.begin(), spatial.end());
    if (layout == TensorLayout::XGCK) r.push_back(g);
    r.push_back(c);
    r.push_back(k);
  }
  return r;
}

Value op_convolution(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 18) throw std::runtime_error("Convolution op expects 18 arguments");
  auto I_or_O = args[0].as_tensor();  // O when deriv_mode is DATA
  auto F_or_O = args[1].as_tensor();  // O when deriv_mode is FILTER
  auto strides = args[2].as_int_tuple_or_empty();
  auto dilations = args[3].as_int_tuple_or_empty();
  auto data_dilations = args[4].as_int_tuple_or_empty();
  auto filter_shape = args[5].as_int_tuple_or_empty();  // spatial filter dims only
  auto groups = args[6].as_int();
  auto autopad_mode = validate<AutoPadMode>(args[7].as_int());
  auto manual_padding = args[8].as_int_tuple_or_empty();
  auto input_layout = validate<TensorLayout>(args[9].as_int());
  auto filter_layout = validate<TensorLayout>(args[10].as_int());
  auto group_layout = validate<GroupLayout>(args[11].as_int());
  auto name = args[13].as_str();
  auto autogroup_mode = validate<AutoGroupMode>(args[14].as_int());
  auto deriv_mode = validate<ConvDerivMode>(args[15].as_int());
  auto result_shape = args[16].as_int_tuple_or_empty();
  const bool infer_result_shape = args[17].as_bool();
  if (name.empty()) name = "conv";

  Tensor I, F, O;
  switch (deriv_mode) {
    case ConvDerivMode::NONE: I = I_or_O; F = F_or_O; break;
    case ConvDerivMode::DATA: O = I_or_O; F = F_or_O; break;
    case ConvDerivMode::FILTER: I = I_or_O; O = F_or_O; break;
    default: throw std::runtime_error("Invalid ConvDerivMode");
  }

  // ---- validation and defaults (ops.cc:671-877)
  const bool is_data_layout = input_layout == TensorLayout::NXC || input_layout == TensorLayout::NCX;
  if (!is_data_layout) throw std::runtime_error("Input tensor layout requested in conv op does not apply to convolution input tensors");
  const bool separate_groups = filter_layout == TensorLayout::GKCX || filter_layout == TensorLayout::XGCK;
  if (!separate_groups && filter_layout != TensorLayout::KCX && filter_layout != TensorLayout::XCK)
    throw std::runtime_error("Filter tensor layout requested in conv op does not apply to convolution filter tensors");
  size_t spatial_rank = strides.size();
  if (spatial_rank == 0) {
    if (I_or_O.rank() < nonspatial_dims(input_layout)) throw std::runtime_error("Convolution data tensor has too few dimensions");
    spatial_rank = I_or_O.rank() - nonspatial_dims(input_layout);
    strides.assign(spatial_rank, 1);
  }
  if (!manual_padding.empty() && autopad_mode != AutoPadMode::EXPLICIT)
    throw std::runtime_error("Autopadding and manual padding both requested for single conv operation");
  auto rank_text = [&](size_t got, const char* what) {
    return "Inconsistent spatial rank in conv op (expecting rank " + std::to_string(spatial_rank) + ", received " +
           std::to_string(got) + "D " + what + ")";
  };
  if (dilations.empty()) dilations.assign(spatial_rank, 1);
  if (dilations.size() != spatial_rank) throw std::runtime_error(rank_text(dilations.size(), "dilations"));
  if (data_dilations.empty()) data_dilations.assign(spatial_rank, 1);
  if (data_dilations.size() != spatial_rank) throw std::runtime_error(rank_text(data_dilations.size(), "data_dilations"));
  if (deriv_mode != ConvDerivMode::DATA && I.rank() != spatial_rank + nonspatial_dims(input_layout))
    throw std::runtime_error("Inconsistent spatial rank in conv op (expected spatial rank " + std::to_string(spatial_rank) +
                             " but input tensor has " + std::to_string(I.rank()) + " dimensions)");
  if (deriv_mode != ConvDerivMode::FILTER && F.rank() != spatial_rank + nonspatial_dims(filter_layout))
    throw std::runtime_error("Inconsistent spatial rank in conv op (expected spatial rank " + std::to_string(spatial_rank) +
                             " but filter tensor has " + std::to_string(F.rank()) + " dimensions)");
  if (!filter_shape.empty() && filter_shape.size() != spatial_rank)
    throw std::runtime_error("Filter shape manually specified with inconsistent rank (expected spatial rank " +
                             std::to_string(spatial_rank) + " but filter_shape has " + std::to_string(filter_shape.size()) + " dimensions)");
  if (separate_groups && group_layout != GroupLayout::SEPARATE)
    throw std::runtime_error("Filter_layout specifies separate groups but group_layout isn't SEPARATE");
  if (!separate_groups && group_layout == GroupLayout::SEPARATE)
    throw std::runtime_error("Filter_layout lacks separate groups but group_layout is SEPARATE");
  if (result_shape.empty()) {
    if (deriv_mode != ConvDerivMode::NONE && !infer_result_shape)
      throw std::runtime_error(
          "Transposed/gradient convolutions require specifying the result_shape. This can be bypassed by setting "
          "infer_result_shape = true, but be warned that infered result shapes do not necessarily match the input "
          "shape used in the forward convolution, as multiple input shapes produce the same output shape.");
  } else if (result_shape.size() != spatial_rank) {
    throw std::runtime_error("Inconsistent spatial rank in conv op (received " + std::to_string(spatial_rank) +
                             " spatial dimensions based on strides but result shape has " + std::to_string(result_shape.size()) +
                             " spatial dims).");
  }
  if (manual_padding.size() > 2 * spatial_rank)
    throw std::runtime_error("Inconsistent spatial rank: operation with " + std::to_string(spatial_rank) + " spatial dimensions had " +
                             std::to_string(manual_padding.size()) + " manual padding values given");
  while (manual_padding.size() < spatial_rank) manual_padding.push_back(0);
  while (manual_padding.size() < 2 * spatial_rank) manual_padding.push_back(manual_padding[manual_padding.size() - spatial_rank]);
  // grouping strategy (ops.cc:811-875)
  switch (autogroup_mode) {
    case AutoGroupMode::UNGROUPED:
      if (groups != 1) throw std::runtime_error("Convolution AutoGroupMode::UNGROUPED requires groups == 1");
      break;
    case AutoGroupMode::AUTO:
      if (group_layout == GroupLayout::NONE) {
        groups = 1;
        autogroup_mode = AutoGroupMode::UNGROUPED;
      }
      if (group_layout == GroupLayout::IN_C)
        throw std::runtime_error("Cannot automatically detect group size of convolution with IN_C GroupLayout");
      break;
    case AutoGroupMode::EXPLICIT:
      if (groups < 1) throw std::runtime_error("Requested grouped convolution with fewer than 1 groups");
      if (groups == 1) autogroup_mode = AutoGroupMode::UNGROUPED;
      if (group_layout == GroupLayout::NONE && groups != 1) throw std::runtime_error("GroupLayout not specified for grouped convolution");
      break;
    case AutoGroupMode::DEPTHWISE:
      if (group_layout == GroupLayout::NONE)
        throw std::runtime_error("Convolution GroupLayout must be specified to use DEPTHWISE AutoGroupMode");
      break;
    default: throw std::runtime_error("Unrecognized AutoGroupMode");
  }

  // ---- dimensions.  TensorDims alias on copy, so a dim bound through one name is bound under every name.
  TensorDim N, CI, CO, G, F_CI, F_CO;
  TensorIndex n("n"), ci("ci"), co("co"), g("g");
  std::vector<TensorDim> I_spatial(spatial_rank), O_spatial(spatial_rank), F_spatial(spatial_rank);
  std::vector<TensorIndex> x, k;
  for (size_t i = 0; i < spatial_rank; ++i) {
    x.emplace_back("x" + std::to_string(i));
    k.emplace_back("k" + std::to_string(i));
  }
  switch (autogroup_mode) {
    case AutoGroupMode::EXPLICIT:
    case AutoGroupMode::UNGROUPED: G = TensorDim(groups); break;
    case AutoGroupMode::DEPTHWISE:
      G = CI;
      if (group_layout == GroupLayout::IN_K || group_layout == GroupLayout::SEPARATE) F_CI = TensorDim(1);
      break;
    case AutoGroupMode::AUTO:  // SEPARATE / IN_K: G is whatever binding the tensors gives it
      break;
    default: break;
  }
  switch (group_layout) {
    case GroupLayout::NONE: F_CO = CO; F_CI = CI; break;
    case GroupLayout::IN_C: F_CI = CI; break;   // CO = F_CO * G below
    case GroupLayout::IN_K: F_CO = CO; break;   // CI = F_CI * G below
    case GroupLayout::SEPARATE: break;          // both below
    default: throw std::runtime_error("Invalid group_layout");
  }
  if (deriv_mode != ConvDerivMode::DATA) I.bind_dims(data_order(input_layout, N, CI, I_spatial));
  if (deriv_mode != ConvDerivMode::FILTER) {
    F.bind_dims(filter_order(filter_layout, G, F_CO, F_CI, F_spatial));
    if (!filter_shape.empty()) {
      std::vector<TensorDim> stated;
      for (int64_t v : filter_shape) stated.emplace_back(v);
      F.bind_dims(filter_order(filter_layout, G, F_CO, F_CI, stated));  // must agree with the tensor's own extents
    }
  }
  if (deriv_mode != ConvDerivMode::NONE) O.bind_dims(data_order(input_layout, N, CO, O_spatial));
  switch (group_layout) {
    case GroupLayout::IN_C: CO = F_CO * G; break;
    case GroupLayout::IN_K: CI = F_CI * G; break;
    case GroupLayout::SEPARATE: CO = F_CO * G; CI = F_CI * G; break;
    default: break;
  }

  // ---- padding and the extents of whichever tensor is being computed (ops.cc:1201-1255)
  std::vector<TensorDim> pad_before;
  if (deriv_mode == ConvDerivMode::NONE) O_spatial.clear();
  if (deriv_mode == ConvDerivMode::DATA) I_spatial.clear();
  for (size_t i = 0; i < spatial_rank; ++i) {
    if (deriv_mode == ConvDerivMode::DATA && result_shape.empty()) {
      auto pr = compute_padding_and_input_size(O_spatial[i], F_spatial[i], strides[i], autopad_mode, manual_padding[i],
                                               manual_padding[i + spatial_rank], dilations[i], data_dilations[i]);
      pad_before.push_back(pr.first);
      I_spatial.push_back(pr.second);
      continue;
    }
    if (deriv_mode == ConvDerivMode::FILTER && result_shape.empty())
      throw std::runtime_error("Result shape inference not yet supported for filter transposed/derivative convolutions");
    TensorDim in_size = deriv_mode == ConvDerivMode::DATA ? TensorDim(result_shape[i]) : I_spatial[i];
    TensorDim f_size = deriv_mode == ConvDerivMode::FILTER ? TensorDim(result_shape[i]) : F_spatial[i];
    auto pr = compute_padding_and_output_size(in_size, f_size, strides[i], autopad_mode, manual_padding[i],
                                              manual_padding[i + spatial_rank], dilations[i], data_dilations[i], false);
    pad_before.push_back(pr.first);
    if (deriv_mode == ConvDerivMode::NONE) O_spatial.push_back(pr.second);
    if (deriv_mode == ConvDerivMode::DATA) I_spatial.push_back(TensorDim(result_shape[i]));
  }

  // ---- index formulas (ops.cc:1342-1450)
  std::vector<Constraint> constraints;
  const bool grouped = group_layout != GroupLayout::NONE;
  std::vector<TensorIndex> I_sp;
  for (size_t i = 0; i < spatial_rank; ++i)
    I_sp.push_back((strides[i] * x[i] + dilations[i] * k[i] - pad_before[i]) / data_dilations[i]);
  auto I_idxs = data_order<TensorIndex>(input_layout, n, grouped ? (CI / G) * g + ci : ci, I_sp);
  auto O_idxs = data_order<TensorIndex>(input_layout, n, grouped ? (CO / G) * g + co : co, x);
  TensorIndex f_co = co, f_ci = ci;
  if (group_layout == GroupLayout::IN_C) {
    f_ci = (CI / G) * g + ci;
    constraints.push_back(ci < CI / G);
  } else if (group_layout == GroupLayout::IN_K) {
    f_co = (CO / G) * g + co;
    constraints.push_back(co < CO / G);
  }
  auto F_idxs = filter_order<TensorIndex>(filter_layout, g, f_co, f_ci, k);

  switch (deriv_mode) {
    case ConvDerivMode::NONE: {
      Tensor R = Contraction(data_order(input_layout, N, CO, O_spatial), O_idxs, name).sum(I(I_idxs) * F(F_idxs)).add_constraints(constraints);
      return Value{R};
    }
    case ConvDerivMode::DATA: {
      Tensor R = Contraction(data_order(input_layout, N, CI, I_spatial), I_idxs, name).sum(O(O_idxs) * F(F_idxs)).add_constraints(constraints);
      return Value{R};
    }
    default: {
      std::vector<TensorDim> stated;
      for (int64_t v : result_shape) stated.emplace_back(v);
      Tensor R = Contraction(filter_order(filter_layout, G, F_CO, F_CI, stated), F_idxs, name).sum(I(I_idxs) * O(O_idxs)).add_constraints(constraints);
      return Value{R};
    }
  }
}

Value op_dot(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("dot expects 3 arguments");
  auto X = args[0].as_tensor();
  auto Y = args[1].as_tensor();
  auto name = args[2].as_str();
  if (name.empty()) name = "dot";
  if (X.dtype() != Y.dtype())
    throw std::runtime_error(std::string("Invalid dtype in dot: X.dtype = '") + to_string(X.dtype()) + "', Y.dtype = '" +
                             to_string(Y.dtype()) + "'");
  if (X.rank() == 1 && Y.rank() == 1) {
    TensorDim I;
    TensorIndex i;
    X.bind_dims(I);
    Y.bind_dims(I);
    Tensor O = Contraction({I}, {i}, name).sum(X(i) * Y(i));
    return Value{O};
  }
  if (1 <= X.rank() && 2 <= Y.rank()) {
    std::vector<TensorDim> X_dims(X.rank()), Y_dims(Y.rank());
    std::vector<TensorIndex> X_idxs(X.rank()), Y_idxs(Y.rank());
    TensorIndex z;
    X_idxs[X.rank() - 1] = z;
    Y_idxs[Y.rank() - 2] = z;
    X.bind_dims(X_dims);
    Y.bind_dims(Y_dims);
    std::vector<TensorDim> O_dims;
    std::vector<TensorIndex> O_idxs;
    for (size_t i = 0; i + 1 < X.rank(); ++i) {
      O_dims.push_back(X_dims[i]);
      O_idxs.push_back(X_idxs[i]);
    }
    for (size_t i = 0; i + 2 < Y.rank(); ++i) {
      O_dims.push_back(Y_dims[i]);
      O_idxs.push_back(Y_idxs[i]);
    }
    O_dims.push_back(Y_dims[Y.rank() - 1]);
    O_idxs.push_back(Y_idxs[Y.rank() - 1]);
    Tensor O = Contraction(O_dims, O_idxs, name).sum(X(X_idxs) * Y(Y_idxs));
    return Value{O};
  }
  throw std::runtime_error("Unsupported dims for dot operation");
}

Value op_maximum(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("maximum expects 2 arguments");
  auto X = args[0].as_tensor(), Y = args[1].as_tensor();
  return Value{select(X < Y, Y, X)};
}
Value op_minimum(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("minimum expects 2 arguments");
  auto X = args[0].as_tensor(), Y = args[1].as_tensor();
  return Value{select(X < Y, X, Y)};
}

Value op_pool(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 10) throw std::runtime_error("PlaidML pool op expects 10 arguments");
  auto I = args[0].as_tensor();
  auto pool_mode = validate<PoolMode>(args[1].as_int());
  auto pool_size = args[2].as_int_tuple();
  auto strides = args[3].as_int_tuple();
  auto autopad_mode = validate<AutoPadMode>(args[4].as_int());
  auto manual_padding = args[5].as_int_tuple();
  auto input_layout = validate<TensorLayout>(args[6].as_int());
  auto include_padding_in_avg = args[7].as_bool();
  auto use_ceil = args[8].as_bool();
  auto name = args[9].as_str();
  if (name.empty()) name = "pool";
  const size_t spatial_rank = pool_size.size();
  if (!manual_padding.empty() && autopad_mode != AutoPadMode::EXPLICIT)
    throw std::runtime_error("Autopadding and manual padding both requested for single pool operation");
  if (strides.size() != spatial_rank) throw std::runtime_error("Inconsistent spatial rank in pool op");
  if (I.rank() != spatial_rank + 2) throw std::runtime_error("Inconsistent spatial rank in pool op");
  if (input_layout != TensorLayout::NXC && input_layout != TensorLayout::NCX)
    throw std::runtime_error("Tensor layout requested in pool op does not apply to pooling");
  if (manual_padding.size() == spatial_rank) {
    auto lo = manual_padding;
    manual_padding.insert(manual_padding.end(), lo.begin(), lo.end());
  }
  manual_padding.resize(2 * spatial_rank, 0);

  TensorDim N, C;
  TensorIndex n("n"), c("c");
  std::vector<TensorDim> X(spatial_rank);
  std::vector<TensorIndex> x, k;
  for (size_t i = 0; i < spatial_rank; ++i) {
    x.emplace_back("x" + std::to_string(i));
    k.emplace_back("k" + std::to_string(i));
  }
  std::vector<TensorDim> I_dims = {N}, O_dims = {N};
  std::vector<TensorIndex> I_idxs = {n}, O_idxs = {n};
  std::vector<Constraint> constraints;
  if (input_layout == TensorLayout::NCX) I_dims.push_back(C);
  for (auto& d : X) I_dims.push_back(d);
  if (input_layout == TensorLayout::NXC) I_dims.push_back(C);
  I.bind_dims(I_dims);
  if (input_layout == TensorLayout::NCX) {
    I_idxs.push_back(c);
    O_dims.push_back(C);
    O_idxs.push_back(c);
  }
  for (size_t i = 0; i < spatial_rank; ++i) {
    O_idxs.push_back(x[i]);
    auto pr = compute_padding_and_output_size(X[i], TensorDim(pool_size[i]), strides[i], autopad_mode, manual_padding[i],
                                              manual_padding[spatial_rank + i], 1, 1, use_ceil);
    O_dims.push_back(pr.second);
    I_idxs.push_back(strides[i] * x[i] + k[i] - pr.first);
    constraints.push_back(k[i] < pool_size[i]);
  }
  if (input_layout == TensorLayout::NXC) {
    I_idxs.push_back(c);
    O_dims.push_back(C);
    O_idxs.push_back(c);
  }
  Contraction O = Contraction(O_dims, O_idxs, name).add_constraints(constraints);
  switch (pool_mode) {
    case PoolMode::MAX: O.max(I(I_idxs)); return Value{Tensor(O)};
    case PoolMode::MIN: O.min(I(I_idxs)); return Value{Tensor(O)};
    case PoolMode::SUM: O.sum(I(I_idxs)); return Value{Tensor(O)};
    case PoolMode::AVG: {
      O.sum(I(I_idxs));
      Tensor S = O;
      if (include_padding_in_avg) {
        int64_t total = 1;
        for (auto s : pool_size) total *= s;
        return Value{S / total};
      }
      auto One = cast(Tensor{1}, I.dtype());
      Tensor Ones = Contraction(I_dims, O_idxs, name).assign(One());
      Tensor Count = Contraction(O_dims, O_idxs, name).sum(Ones(I_idxs)).add_constraints(constraints);
      return Value{S / Count};
    }
    default: throw std::runtime_error("Unrecognized pool_mode in pool op");
  }
}

Value op_relu(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 5) throw std::runtime_error("relu expects 5 arguments");
  Tensor I = args[0].as_tensor();
  Value alpha = args[1], max_value = args[2], threshold = args[3];
  auto name = args[4].as_str();
  if (name.empty()) name = "relu";
  const double T = threshold.is_none() ? 0.0 : threshold.as_float();
  if ((alpha.is_none() || (alpha.is_float() && alpha.as_float() == 0.0)) && max_value.is_none() && T == 0.0)
    return Value{edsl::relu(I, name)};
  Tensor A = alpha.is_none() ? Tensor(0.0) : alpha.as_tensor();
  Tensor O = select(I < T, cast(A * (I - T), I.dtype()), I);
  if (!max_value.is_none()) {
    Tensor M = cast(max_value.as_tensor(), I.dtype());
    O = select(O < M, O, M);
  }
  return Value{O};
}

Value op_softmax(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("softmax expects 3 arguments");
  auto I = args[0].as_tensor();
  int64_t axis = args[1].as_int();
  auto name = args[2].as_str();
  if (name.empty()) name = "softmax";
  const int64_t ndims = static_cast<int64_t>(I.rank());
  if (axis < 0) axis += ndims;
  if (axis < 0 || axis >= ndims) throw std::runtime_error("Axis out of range for softmax op");
  if (axis != ndims - 1) throw std::runtime_error("softmax over a non-trailing axis is not supported by this backend");
  std::vector<TensorDim> I_dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> R_dims = I_dims;
  std::vector<TensorIndex> R_idxs = I_idxs;
  R_dims[axis] = TensorDim(1);
  R_idxs[axis] = TensorIndex(static_cast<int64_t>(0));
  Tensor M = Contraction(R_dims, R_idxs, name).max(I(I_idxs));
  auto E = exp(I - M);
  Tensor Nn = Contraction(R_dims, R_idxs, name).sum(E(I_idxs));
  return Value{E / Nn};
}

size_t normalize_axis(int64_t axis, size_t ndims, const char* what) {
  const int64_t n = static_cast<int64_t>(ndims);
  if (axis < -n || axis >= n)
    throw std::runtime_error(std::string("axis out of range in ") + what + ": " + std::to_string(axis) + " for a tensor of rank " +
                             std::to_string(ndims));
  return static_cast<size_t>(axis < 0 ? axis + n : axis);
}

std::vector<int64_t> int_or_ints(const Value& v) {
  if (v.is_int()) return {v.as_int()};
  return v.as_int_tuple();
}

Value op_abs(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 1) throw std::runtime_error("abs expects 1 argument");
  auto I = args[0].as_tensor();
  return Value{select(I < 0., -I, I)};
}

Tensor concatenate(std::vector<Tensor> tensors, int64_t raw_axis) {
  if (tensors.empty()) throw std::runtime_error("The concatenate op requires at least one input tensor");
  const size_t ndims = tensors[0].rank();
  const size_t axis = normalize_axis(raw_axis, ndims, "concatenate");
  // every input is placed at its offset along the axis of an otherwise empty result; the results are added
  std::vector<TensorDim> dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  std::vector<TensorDim> axis_dims(tensors.size());
  std::vector<TensorDim> offsets{TensorDim(0)};
  for (size_t i = 0; i < tensors.size(); ++i) {
    if (tensors[i].rank() != ndims) throw std::runtime_error("concatenate: inputs differ in rank");
    dims[axis] = axis_dims[i];
    tensors[i].bind_dims(dims);
    offsets.push_back(axis_dims[i] + offsets.back());
  }
  dims[axis] = offsets.back();
  Tensor result;
  for (size_t i = 0; i < tensors.size(); ++i) {
    std::vector<TensorIndex> O_idxs = I_idxs;
    O_idxs[axis] = I_idxs[axis] + offsets[i];
    Tensor R = Contraction(dims, O_idxs, "concatenate").assign(tensors[i](I_idxs));
    result = i == 0 ? R : result + R;
  }
  return result;
}

Value op_concatenate(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("concatenate expects 2 arguments");
  std::vector<Tensor> tensors;
  for (const auto& t : args[0].as_tuple()) tensors.push_back(t.as_tensor());
  return Value{concatenate(tensors, args[1].as_int())};
}

Value op_cumsum(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("cumsum expects 3 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  const size_t axis = normalize_axis(args[1].as_int(), ndims, "cumsum");
  const bool exclusive = args[2].as_bool();
  std::vector<TensorDim> dims(ndims);
  I.bind_dims(dims);
  std::vector<TensorIndex> O_idxs(ndims);
  std::vector<TensorIndex> I_idxs = O_idxs;
  TensorIndex back;
  I_idxs[axis] = exclusive ? O_idxs[axis] - back - 1 : O_idxs[axis] - back;
  Tensor O = Contraction(dims, O_idxs, "cumsum").sum(I(I_idxs)).add_constraint(back < dims[axis]);
  return Value{O};
}

Value op_elu(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("elu expects 2 arguments");
  auto I = args[0].as_tensor();
  if (args[1].is_float()) {
    const double alpha = args[1].as_float();
    return Value{select(I < 0., alpha * exp(I) - alpha, I)};
  }
  if (args[1].is_int()) {
    const int64_t alpha = args[1].as_int();
    return Value{select(I < 0., alpha * exp(I) - alpha, I)};
  }
  throw std::runtime_error("Unexpected type for alpha in elu");
}

Value op_explicit_padding(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() < 5) throw std::runtime_error("explicit_padding expects 5 arguments");
  auto I = args[0].as_tensor();
  auto lo = args[1].as_int_tuple();
  auto hi = args[2].as_int_tuple();
  const auto mode = validate<plaidml::op::PadMode>(args[3].as_int());
  const size_t ndims = I.rank();
  if (lo.size() != ndims || hi.size() != ndims)
    throw std::runtime_error("Inconsistent shapes in explicit_padding op (one lower and one upper padding per dimension expected)");
  std::vector<TensorDim> X(ndims);
  std::vector<TensorIndex> x(ndims);
  I.bind_dims(X);
  if (mode == plaidml::op::PadMode::CONSTANT) {
    std::vector<TensorDim> O_dims;
    std::vector<TensorIndex> O_idxs;
    for (size_t i = 0; i < ndims; ++i) {
      O_dims.push_back(X[i] + lo[i] + hi[i]);
      O_idxs.push_back(x[i] + lo[i]);
    }
    Tensor O = Contraction(O_dims, O_idxs, "explicit_padding").assign(I(x)).init(args[4].as_tensor());
    return Value{O};
  }
  if (mode == plaidml::op::PadMode::EDGE) {
    // dimension by dimension: the first / last slice repeated lo / hi times, joined around the tensor so far
    Tensor O = I;
    for (size_t i = 0; i < ndims; ++i) {
      std::vector<TensorDim> D(ndims);
      O.bind_dims(D);
      std::vector<TensorIndex> dst(ndims);
      std::vector<TensorIndex> src_lo = dst, src_hi = dst;
      src_lo[i] = TensorIndex(static_cast<int64_t>(0));
      src_hi[i] = D[i] - TensorIndex(static_cast<int64_t>(1));
      std::vector<TensorDim> lo_dims = D, hi_dims = D;
      lo_dims[i] = TensorDim(lo[i]);
      hi_dims[i] = TensorDim(hi[i]);
      Tensor Lo = Contraction(lo_dims, dst, "explicit_padding").assign(O(src_lo));
      Tensor Hi = Contraction(hi_dims, dst, "explicit_padding").assign(O(src_hi));
      O = concatenate({Lo, O, Hi}, static_cast<int64_t>(i));
    }
    return Value{O};
  }
  throw std::runtime_error("Unimplemented padding mode (only CONSTANT and EDGE exist, as in the reference)");
}

Value op_flip(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("flip expects 2 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  std::vector<int64_t> raw;
  if (args[1].is_none()) {
    for (size_t i = 0; i < ndims; ++i) raw.push_back(static_cast<int64_t>(i));
  } else {
    raw = int_or_ints(args[1]);
  }
  std::vector<TensorDim> dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  std::vector<TensorIndex> O_idxs = I_idxs;
  I.bind_dims(dims);
  for (int64_t a : raw) {
    const size_t axis = normalize_axis(a, ndims, "flip");
    O_idxs[axis] = dims[axis] - 1 - I_idxs[axis];
  }
  Tensor O = Contraction(dims, O_idxs, "flip").assign(I(I_idxs));
  return Value{O};
}

Value op_hard_sigmoid(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("hard_sigmoid expects 2 arguments");
  auto I = args[0].as_tensor();
  const double slope = args[1].as_float();
  if (slope <= 0) throw std::runtime_error("hard_sigmoid expects positive slope, received " + std::to_string(slope));
  const double hi_cusp = 1. / (2. * slope), lo_cusp = -hi_cusp;
  auto lo = cast(Tensor(0.), I.dtype());
  auto hi = cast(Tensor(1.), I.dtype());
  return Value{select(I < lo_cusp, lo, select(I > hi_cusp, hi, slope * I + 0.5))};
}

Value op_variance(const Value& value);

// all / any (plaidml/op/lib/ops.cc:450-503): the input as 0 / 1 in its own type, multiplied (all) or summed and
// tested (any) over the axes, as UINT8.
Tensor truth_of(const Tensor& I, Tensor* zero, Tensor* one) {
  *one = cast(Tensor(int64_t{1}), I.dtype());
  *zero = cast(Tensor(int64_t{0}), I.dtype());
  return select(I == 0, *zero, *one);
}

Value op_all(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("all expects 3 arguments");
  auto I = args[0].as_tensor();
  Tensor zero, one;
  Tensor T = truth_of(I, &zero, &one);
  if (I.rank() == 0 || (args[1].is_tuple() && args[1].as_tuple().empty())) return Value{cast(T, DType::UINT8)};
  AggregationAxes ag(I.rank(), args[1], args[2].as_bool());
  I.bind_dims(ag.src_dims);
  Tensor O = Contraction(ag.dst_dims, ag.dst_idxs, "all").product(T(ag.src_idxs));
  return Value{cast(O, DType::UINT8)};
}

Value op_any(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("any expects 3 arguments");
  auto I = args[0].as_tensor();
  Tensor zero, one;
  Tensor T = truth_of(I, &zero, &one);
  if (I.rank() == 0 || (args[1].is_tuple() && args[1].as_tuple().empty())) return Value{cast(T, DType::UINT8)};
  AggregationAxes ag(I.rank(), args[1], args[2].as_bool());
  I.bind_dims(ag.src_dims);
  Tensor S = Contraction(ag.dst_dims, ag.dst_idxs, "any").sum(T(ag.src_idxs));
  return Value{cast(select(S == 0, zero, one), DType::UINT8)};
}

// plaidml/op/lib/ops.cc:523-544: predictions clipped to [eps, 1 - eps], then -T log P - (1 - T) log(1 - P)
Value op_binary_crossentropy(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("binary_crossentropy expects 3 arguments");
  auto T = args[0].as_tensor();
  const double epsilon = args[2].as_float();
  if (epsilon < 0. || epsilon >= 0.5)
    throw std::runtime_error("The epsilon used in binary_crossentropy must be between 0 and 0.5, received " + std::to_string(epsilon));
  auto P = op_clip(make_tuple(args[1], Value{epsilon}, Value{1. - epsilon})).as_tensor();
  return Value{-T * log(P) - (1 - T) * log(1 - P)};
}

// plaidml/op/lib/ops.cc:546-582: input dimension i becomes output dimension axes[i]; an input extent of 1 repeats
Value op_broadcast(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3)
    throw std::runtime_error("PlaidML broadcast op expects 3 arguments (received " + std::to_string(args.size()) + ")");
  auto I = args[0].as_tensor();
  auto axes = args[2].as_int_tuple_or_empty();
  if (I.rank() != axes.size())
    throw std::runtime_error("Mismatched broadcast axes (received " + std::to_string(axes.size()) +
                             " broadcast axes for input tensor of rank " + std::to_string(I.rank()) + ")");
  const auto in_sizes = I.compute_shape().sizes();
  auto target = args[1].as_int_tuple_or_empty();
  std::vector<TensorDim> O_dims(target.begin(), target.end());
  std::vector<TensorDim> I_dims(I.rank());
  I.bind_dims(I_dims);
  std::vector<TensorIndex> O_idxs(target.size()), I_idxs;
  for (size_t i = 0; i < axes.size(); ++i) {
    if (in_sizes[i] == 1) {
      I_idxs.emplace_back(0);
    } else {
      if (axes[i] < 0 || axes[i] >= static_cast<int64_t>(target.size())) throw std::out_of_range("broadcast axis out of range");
      I_idxs.push_back(O_idxs[axes[i]]);
    }
  }
  Tensor O = Contraction(O_dims, O_idxs, "broadcast").assign(I(I_idxs));
  return Value{O};
}

// plaidml/op/lib/ops.cc:1469-1488
Value op_cumprod(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("cumprod expects 2 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  const size_t axis = normalize_axis(args[1].as_int(), ndims, "cumprod");
  std::vector<TensorDim> dims(ndims);
  I.bind_dims(dims);
  std::vector<TensorIndex> O_idxs(ndims);
  std::vector<TensorIndex> I_idxs = O_idxs;
  TensorIndex back;
  I_idxs[axis] = O_idxs[axis] - back;
  Tensor O = Contraction(dims, O_idxs, "cumprod").product(I(I_idxs)).add_constraint(back < dims[axis]);
  return Value{O};
}

// plaidml/op/lib/ops.cc:2505-2530: sqrt(sum of squares over the axes (kept), + eps or max(., eps))
Value op_l2norm(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 4) throw std::runtime_error("norm expects 4 arguments");
  auto I = args[0].as_tensor();
  const double epsilon = args[2].as_float();
  const auto mode = validate<EpsMode>(args[3].as_int());
  Tensor X = reduce(make_tuple(Value{I * I}, args[1], Value{true}), "sum", PLAIDML_AGG_OP_SUM).as_tensor();
  switch (mode) {
    case EpsMode::ADD: X = X + epsilon; break;
    case EpsMode::MAX: X = op_maximum(make_tuple(Value{X}, Value{cast(Tensor(epsilon), X.dtype())})).as_tensor(); break;
    default: throw std::runtime_error("Unrecognized eps_mode in l2norm op");
  }
  return Value{sqrt(X)};
}

// plaidml/op/lib/ops.cc:129-160, 1920-1941: I / (alpha * sum of squares over a centred window + eps) ^ beta
Value op_lrn(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 6) throw std::runtime_error("lrn expects 6 arguments");
  auto I = args[0].as_tensor();
  const auto widths = args[1].as_int_tuple_or_empty();
  const auto in_axes = args[2].as_int_tuple_or_empty();
  const double alpha = args[3].as_float(), beta = args[4].as_float(), epsilon = args[5].as_float();
  const size_t ndims = I.rank();
  std::set<int64_t> axes;
  for (int64_t a : in_axes) {
    if (a < 0) a += ndims;
    if (a < 0 || a >= static_cast<int64_t>(ndims)) throw std::out_of_range("axis out of range: " + std::to_string(a));
    axes.insert(a);
  }
  if (axes.size() != widths.size())
    throw std::runtime_error("Inconsistent axis count and window width count in LRN (" + std::to_string(axes.size()) + " vs " +
                             std::to_string(widths.size()) + ")");
  std::vector<TensorDim> dims(ndims);
  I.bind_dims(dims);
  std::vector<TensorIndex> dst(ndims);
  std::vector<TensorIndex> src = dst;
  std::vector<TensorIndex> win(widths.size());
  std::vector<Constraint> cons;
  size_t k = 0;
  for (int64_t a : axes) {
    cons.push_back(win[k] < widths[k]);
    src[a] = dst[a] + win[k] - widths[k] / 2;
    ++k;
  }
  Tensor sq = I * I;
  Tensor local = Contraction(dims, dst, "lrn").sum(sq(src)).add_constraints(cons);
  return Value{I / pow(alpha * local + epsilon, Tensor(beta))};
}

// plaidml/op/lib/ops.cc:2469-2503
Value op_mvn(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 6) throw std::runtime_error("mvn expects 6 arguments");
  auto I = args[0].as_tensor();
  Value axes = args[1];
  const bool normalize_variance = args[2].as_bool();
  const double epsilon = args[3].as_float();
  const bool across_channels = args[4].as_bool();
  const std::string layout = args[5].as_str();
  if (axes.is_none()) {
    if (layout.empty()) throw std::runtime_error("Either axes or layout must be specified for MVN");
    std::vector<Value> raw;
    for (size_t i = 0; i < layout.size(); ++i) {
      if (layout[i] == 'N') continue;
      if (layout[i] == 'C' && !across_channels) continue;
      raw.emplace_back(static_cast<int64_t>(i));
    }
    axes = Value(raw);
  }
  Tensor R = I - reduce(make_tuple(args[0], axes, Value{true}), "mean", PLAIDML_AGG_OP_SUM).as_tensor();
  if (normalize_variance) {
    Tensor stdev = sqrt(op_variance(make_tuple(args[0], axes, Value{true})).as_tensor());
    R = R / op_maximum(make_tuple(Value{stdev}, Value{cast(Tensor(epsilon), I.dtype())})).as_tensor();
  }
  return Value{R};
}

// plaidml/op/lib/ops.cc:2730-2780: blocks of stride x stride pixels move between the spatial and the channel
// dimensions; the contraction is written in NCHW and seen through a lens for other layouts
Value op_reorg_yolo(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 4)
    throw std::runtime_error("PlaidML reorg_yolo op expects 4 arguments (received " + std::to_string(args.size()) + ")");
  auto I = args[0].as_tensor();
  const int64_t stride = args[1].as_int();
  const bool decrease = args[2].as_bool();
  const std::string layout = args[3].as_str();
  if (I.rank() != 4)
    throw std::runtime_error("PlaidML reorg_yolo op expects I to have 4 dimensions (received " + std::to_string(I.rank()) + ")");
  TensorLens lens(layout, "NCHW");
  I = I.use(lens);
  TensorDim N, C, H, W;
  I.bind_dims(N, C, H, W);
  TensorIndex b, i, j, k, x, y;
  auto h = j * stride + y;
  auto w = i * stride + x;
  Tensor O;
  if (decrease) {
    auto C_out = C / (stride * stride);
    auto c = k + ((x + y * stride) * C_out);
    O = Contraction(lens, "reorg_yolo").outShape(N, C_out, H * stride, W * stride).outAccess(b, k, h, w).assign(I(b, c, j, i))
            .add_constraint(y < stride).add_constraint(x < stride);
  } else {
    auto C_out = C * (stride * stride);
    auto c = k + ((x + y * stride) * C);
    O = Contraction(lens, "reorg_yolo").outShape(N, C_out, H / stride, W / stride).outAccess(b, c, j, i).assign(I(b, k, h, w))
            .add_constraint(y < stride).add_constraint(x < stride);
  }
  return Value{O};
}

// plaidml/op/lib/ops.cc:2888-2904: the forward pass is the identity
Value op_scale_gradient(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("scale_gradient expects 2 arguments");
  return Value{args[0].as_tensor()};
}

// plaidml/op/lib/ops.cc:2917-3047: per axis an integer (the axis disappears) or (start, stop, step) with None
// defaults and negative values counted from the end; no clamping, as in the reference
Value op_slice(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("slice expects 2 arguments");
  auto I = args[0].as_tensor();
  auto slices = args[1].as_tuple();
  const size_t ndims = I.rank();
  if (ndims == 0) return Value{I};
  if (slices.size() != ndims)
    throw std::runtime_error(std::to_string(slices.size()) + " slice axes provided to slice " + std::to_string(ndims) + "-dimensional tensor");
  std::vector<TensorDim> I_dims(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorIndex> O_idxs, I_idxs;
  std::vector<TensorDim> O_dims;
  for (size_t i = 0; i < ndims; ++i) {
    if (slices[i].is_int()) {
      const int64_t at = slices[i].as_int();
      TensorIndex idx(at);
      if (at < 0) idx = idx + I_dims[i];
      I_idxs.push_back(idx);
      continue;
    }
    if (!slices[i].is_tuple()) throw std::runtime_error("Attempted to define slice with invalid type");
    auto sl = slices[i].as_tuple();
    if (sl.size() != 3) throw std::runtime_error("Attempted to slice with " + std::to_string(sl.size()) + " entries, 3 required");
    const int64_t step = sl[2].is_none() ? 1 : sl[2].as_int();
    if (step == 0) throw std::runtime_error("Cannot slice with step size 0");
    TensorDim start, stop;
    if (sl[0].is_none()) {
      start = step > 0 ? TensorDim(0) : I_dims[i] - 1;
    } else {
      const int64_t v = sl[0].as_int();
      start = v < 0 ? I_dims[i] + v : TensorDim(v);
    }
    if (sl[1].is_none()) {
      stop = step > 0 ? I_dims[i] : TensorDim(-1);
    } else {
      const int64_t v = sl[1].as_int();
      stop = v < 0 ? I_dims[i] + v : TensorDim(v);
    }
    const int64_t to_ceil = step > 0 ? step - 1 : step + 1;
    O_dims.push_back((stop - start + to_ceil) / step);
    TensorIndex o;
    O_idxs.push_back(o);
    I_idxs.push_back(start + step * o);
  }
  Tensor O = Contraction(O_dims, O_idxs, "slice").assign(I(I_idxs));
  return Value{O};
}

Value op_prod(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("prod expects 3 arguments");
  auto I = args[0].as_tensor();
  if (I.rank() == 0) return Value{I};
  auto axes = args[1];
  if (axes.is_tuple() && axes.as_tuple().empty()) return Value{I};
  AggregationAxes ag(I.rank(), axes, args[2].as_bool());
  I.bind_dims(ag.src_dims);
  Tensor O = Contraction(ag.dst_dims, ag.dst_idxs, "prod").product(I(ag.src_idxs));
  return Value{O};
}

Value op_repeat(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("repeat expects 3 arguments");
  auto I = args[0].as_tensor();
  TensorDim repeats;
  if (args[1].is_int())
    repeats = TensorDim(args[1].as_int());
  else if (args[1].is_dim())
    repeats = args[1].as_dim();
  else
    throw std::runtime_error("Repeat only accepts int or TensorDim for repeats parameter");
  const size_t ndims = I.rank();
  const size_t axis = normalize_axis(args[2].as_int(), ndims, "repeat");
  std::vector<TensorDim> I_dims(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims = I_dims;
  O_dims[axis] = repeats * I_dims[axis];
  std::vector<TensorIndex> I_idxs(ndims);
  std::vector<TensorIndex> O_idxs = I_idxs;
  TensorIndex inner;
  O_idxs[axis] = repeats * I_idxs[axis] + inner;
  Tensor O = Contraction(O_dims, O_idxs, "repeat").assign(I(I_idxs)).add_constraint(inner < repeats);
  return Value{O};
}

Value op_reshape(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("reshape expects 2 arguments");
  auto I = args[0].as_tensor();
  std::vector<TensorDim> I_dims(I.rank());
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims;
  size_t fill_dim = 0;
  bool fill = false;
  auto target = args[1].as_tuple();
  auto match = [&](size_t i) {
    if (i >= I_dims.size())
      throw std::runtime_error("matching dimension requested at " + std::to_string(i + 1) + " from " + std::to_string(I_dims.size()) +
                               "-dimensional tensor");
    O_dims.push_back(I_dims[i]);
  };
  for (size_t i = 0; i < target.size(); ++i) {
    if (target[i].is_int()) {
      const int64_t d = target[i].as_int();
      if (d == plaidml::op::AUTO_DIM_MATCH) {
        match(i);
      } else if (d == plaidml::op::AUTO_DIM_FILL) {
        if (fill) throw std::runtime_error("at most one dimension's size may be inferred");
        fill = true;
        fill_dim = i;
        O_dims.emplace_back(1);
      } else {
        O_dims.emplace_back(d);
      }
    } else if (target[i].is_dim()) {
      O_dims.push_back(target[i].as_dim());
    } else if (target[i].is_none()) {
      match(i);
    } else {
      throw std::runtime_error("reshape: a dimension must be an integer, a TensorDim or None");
    }
  }
  if (fill) {
    TensorDim num(1), den(1);
    for (const auto& d : I_dims) num = d * num;
    for (const auto& d : O_dims) den = d * den;
    O_dims[fill_dim] = TensorDim(num / den);
  }
  return Value{edsl::reshape(I, O_dims)};
}

Value op_sigmoid(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 1) throw std::runtime_error("sigmoid expects 1 argument");
  auto I = args[0].as_tensor();
  return Value{1.0 / (1.0 + exp(-I))};
}

Value op_spatial_padding(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 4) throw std::runtime_error("spatial_padding expects 4 arguments");
  auto I = args[0].as_tensor();
  auto lo = args[1].as_int_tuple();
  auto hi = args[2].as_int_tuple();
  const auto layout = validate<TensorLayout>(args[3].as_int());
  if (layout != TensorLayout::NXC && layout != TensorLayout::NCX)
    throw std::runtime_error("spatial_padding: only the NXC and NCX layouts are supported by this backend");
  const size_t ndims = I.rank();
  if (ndims < 3) throw std::runtime_error("Insufficient spatial rank in spatial_padding op (at least 1 spatial dim required)");
  const size_t spatial = ndims - 2;
  if (lo.size() != spatial || hi.size() != spatial)
    throw std::runtime_error("Inconsistent spatial rank in spatial_padding op (one lower and one upper padding per spatial dim expected)");
  const size_t first = layout == TensorLayout::NXC ? 1 : 2;  // position of the first spatial dimension
  std::vector<TensorDim> I_dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims = I_dims;
  std::vector<TensorIndex> O_idxs = I_idxs;
  for (size_t i = 0; i < spatial; ++i) {
    O_dims[first + i] = I_dims[first + i] + lo[i] + hi[i];
    O_idxs[first + i] = I_idxs[first + i] + lo[i];
  }
  Tensor O = Contraction(O_dims, O_idxs, "spatial_padding").assign(I(I_idxs));
  return Value{O};
}

Value op_square(const Value& value) {
  auto x = value.is_tuple() ? value.as_tuple().at(0).as_tensor() : value.as_tensor();
  return Value{x * x};
}

Value op_squeeze(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("Squeeze expects 2 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  std::vector<TensorDim> I_dims(ndims);
  I.bind_dims(I_dims);
  std::set<size_t> axes;
  for (int64_t a : int_or_ints(args[1])) axes.insert(normalize_axis(a, ndims, "squeeze"));
  std::vector<TensorDim> O_dims;
  for (size_t i = 0; i < ndims; ++i)
    if (!axes.count(i)) O_dims.push_back(I_dims[i]);
  return Value{edsl::reshape(I, O_dims)};
}

Value op_tile(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("Tile expects 2 arguments");
  auto I = args[0].as_tensor();
  auto reps = args[1].as_int_tuple();
  const size_t ndims = I.rank();
  if (reps.empty()) throw std::runtime_error("No tiling factors provided to tile operation");
  while (reps.size() < ndims) reps.push_back(1);
  if (reps.size() > ndims) throw std::runtime_error("More tiling factors provided to tile operation than tensor dimensions");
  std::vector<TensorDim> I_dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims;
  std::vector<TensorIndex> O_idxs;
  for (size_t i = 0; i < ndims; ++i) {
    O_dims.push_back(I_dims[i] * reps[i]);
    O_idxs.push_back(TensorIndex() * I_dims[i] + I_idxs[i]);
  }
  Tensor O = Contraction(O_dims, O_idxs, "tile").assign(I(I_idxs));
  return Value{O};
}

Value op_transpose(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("Transpose expects 2 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  std::vector<int64_t> pattern;
  if (args[1].is_none()) {
    for (size_t i = 0; i < ndims; ++i) pattern.push_back(static_cast<int64_t>(ndims - 1 - i));
  } else if (args[1].is_tuple()) {
    pattern = args[1].as_int_tuple();
  } else {
    throw std::runtime_error("Transpose 2nd argument must be none or integer tuple");
  }
  if (pattern.size() != ndims) throw std::runtime_error("Transpose pattern must name every dimension once");
  for (int64_t i : pattern)
    if (i < 0 || static_cast<size_t>(i) >= ndims)
      throw std::runtime_error("Transpose of nonexistent axis " + std::to_string(i) + " requested (input has " + std::to_string(ndims) +
                               " dimensions)");
  std::vector<TensorDim> I_dims(ndims);
  std::vector<TensorIndex> I_idxs(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims;
  std::vector<TensorIndex> O_idxs;
  for (size_t i = 0; i < ndims; ++i) {
    O_dims.push_back(I_dims[pattern[i]]);
    O_idxs.push_back(I_idxs[pattern[i]]);
  }
  Tensor O = Contraction(O_dims, O_idxs, "transpose").assign(I(I_idxs));
  return Value{O};
}

Value op_unsqueeze(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 2) throw std::runtime_error("unsqueeze expects 2 arguments");
  auto I = args[0].as_tensor();
  const size_t ndims = I.rank();
  auto raw = int_or_ints(args[1]);
  std::set<size_t> axes;
  for (int64_t a : raw) axes.insert(normalize_axis(a, ndims + raw.size(), "unsqueeze"));
  std::vector<TensorDim> I_dims(ndims);
  I.bind_dims(I_dims);
  std::vector<TensorDim> O_dims;
  size_t src = 0;
  for (size_t i = 0; i < ndims + axes.size(); ++i) {
    if (axes.count(i))
      O_dims.emplace_back(1);
    else if (src < ndims)
      O_dims.push_back(I_dims[src++]);
  }
  if (src != ndims) throw std::runtime_error("Unsqueeze did not replicate entirety of input into output");
  return Value{edsl::reshape(I, O_dims)};
}

Value op_variance(const Value& value) {
  // the uncorrected sample variance (denominator n)
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("Variance expects 3 arguments");
  auto I = args[0].as_tensor();
  auto axes = args[1];
  if (I.rank() == 0) return Value{Tensor(static_cast<int64_t>(0))};
  if (axes.is_tuple() && axes.as_tuple().empty()) throw std::runtime_error("Variance expects nonempty axis list");
  Tensor Mean = reduce(make_tuple(I, axes, true), "mean", PLAIDML_AGG_OP_SUM).as_tensor();
  AggregationAxes ag(I.rank(), axes, args[2].as_bool());
  I.bind_dims(ag.src_dims);
  Tensor D2 = (I - Mean) * (I - Mean);
  Tensor S = Contraction(ag.dst_dims, ag.dst_idxs, "variance").sum(D2(ag.src_idxs));
  Tensor denom(1);
  for (size_t a : ag.axes) denom = denom * ag.src_dims.at(a);
  return Value{S / denom};
}

// ---- operations built on the special intrinsics ------------------------------------------------------------
Value int_tuple(const std::vector<int64_t>& v) {
  std::vector<Value> vals;
  for (int64_t x : v) vals.emplace_back(x);
  return Value(vals);
}
Tensor unsqueeze_at(const Tensor& t, int64_t axis) { return op_unsqueeze(make_tuple(Value{t}, int_tuple({axis}))).as_tensor(); }
Tensor squeeze_last(const Tensor& t) { return op_squeeze(make_tuple(Value{t}, int_tuple({-1}))).as_tensor(); }

// plaidml/op/lib/ops.cc:1728-1801.  Without interpolation this is the ND mode of the gather intrinsic.  LINEAR
// (floating coordinates) pads the addressed dimensions with two zeros on each side and sums the 2^k corners of
// the surrounding cell, each gathered with integer coordinates and weighted by the opposite distances.
Value op_gatherND(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 4) throw std::runtime_error("gatherND expects 4 arguments");
  auto I = args[0].as_tensor();
  auto idx = args[1].as_tensor();
  const int64_t batch_dims = args[2].as_int();
  const int64_t I_rank = static_cast<int64_t>(I.rank());
  const auto idx_shape = idx.compute_shape().sizes();
  if (idx_shape.empty()) throw std::runtime_error("gatherND needs indices of at least one dimension");
  const int64_t idx_dims = idx_shape.back();
  if (idx_dims + batch_dims > I_rank)
    throw std::runtime_error("Invalid Indices: Data(shape: '" + I.compute_shape().str() + "'), Indices(shape: '" +
                             idx.compute_shape().str() + "'), BatchDims('" + std::to_string(batch_dims) + "')");
  const auto mode = static_cast<InterpolationMode>(args[3].as_int());
  if (mode == InterpolationMode::NONE) return Value{gatherBuilder(I, idx, static_cast<uint64_t>(batch_dims), mode).build()};
  if (mode != InterpolationMode::LINEAR) throw std::runtime_error("Unsupported InterpolationMode in gatherND");
  const int64_t pad_length = 2;
  std::vector<int64_t> pads(I_rank, 0);
  for (int64_t i = 0; i < idx_dims; ++i) pads[i + batch_dims] = pad_length;
  Tensor X = op_explicit_padding(make_tuple(Value{I}, int_tuple(pads), int_tuple(pads),
                                            Value{static_cast<int64_t>(plaidml::op::PadMode::CONSTANT)}, Value{Tensor(int64_t{0})}))
                 .as_tensor();
  Tensor Y = idx + pad_length;
  if (static_cast<int64_t>(idx_shape.size()) - batch_dims != 2)
    throw std::runtime_error(
        " Indices dimension should be batch_dims plus two in interpolated gatherND, please reshape indices to satisfy this "
        "requirement.");
  Tensor Y_float = cast(Y, DType::FLOAT32);
  std::vector<Tensor> dims, lower, upper;
  for (int64_t i = 0; i < idx_dims; ++i) {
    Tensor dim = gather(Y_float, static_cast<int>(i)).axis(-1);
    dims.push_back(dim);
    lower.push_back(floor(dim));
    upper.push_back(floor(dim) + 1.0);
  }
  Tensor ZERO = cast(index({TensorDim(1)}, 0), DType::FLOAT32);
  Tensor result = ZERO;
  const int64_t corners = int64_t{1} << idx_dims;
  for (int64_t corner = 0; corner < corners; ++corner) {
    std::vector<Tensor> at;
    Tensor coeff = ZERO + 1;
    for (int64_t k = 0, j = corner; k < idx_dims; ++k, j /= 2) {
      const bool high = (j % 2) != 0;
      at.push_back(high ? upper[k] : lower[k]);
      coeff = high ? coeff * squeeze_last(dims[k] - lower[k]) : coeff * squeeze_last(upper[k] - dims[k]);
    }
    Tensor at_int = cast(concatenate(at, -1), DType::INT32);
    Tensor vertex = gatherBuilder(X, at_int, static_cast<uint64_t>(batch_dims), InterpolationMode::NONE).build();
    std::vector<int64_t> axes;
    for (size_t i = 0; i < coeff.rank(); ++i) axes.push_back(static_cast<int64_t>(i));
    Tensor spread = op_broadcast(make_tuple(Value{coeff}, int_tuple(vertex.compute_shape().sizes()), int_tuple(axes))).as_tensor();
    result = result + vertex * spread;
  }
  return Value{result};
}

// plaidml/op/lib/ops.cc:3100-3127: the sorted values are gathered with full coordinates whose `axis` entry is the
// argsort and whose other entries are the element's own position
Tensor sorted_by(const Tensor& I, const Tensor& order, int64_t axis) {
  const int64_t ndims = static_cast<int64_t>(I.rank());
  std::vector<TensorDim> dims(order.rank());
  order.bind_dims(dims);
  std::vector<Tensor> coords;
  for (int64_t i = 0; i < ndims; ++i) coords.push_back(unsqueeze_at(i == axis ? order : index(dims, static_cast<size_t>(i)), ndims));
  return gatherBuilder(I, concatenate(coords, -1), 0, InterpolationMode::NONE).build();
}

Value op_sort(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 3) throw std::runtime_error("sort expects 3 arguments");
  auto I = args[0].as_tensor();
  const int64_t raw_direction = args[2].as_int();
  if (raw_direction != 0 && raw_direction != 1) throw std::runtime_error("Invalid enumeration value in operation arguments");
  const auto direction = static_cast<SortDirection>(raw_direction);
  const int64_t axis = static_cast<int64_t>(normalize_axis(args[1].as_int(), I.rank(), "sort"));
  return Value{sorted_by(I, argsort(I, static_cast<int>(axis), direction), axis)};
}

// plaidml/op/lib/ops.cc:2420-2467: the first k of the sorted values and positions; sort type INDEX re-orders those k
// by position
Value op_topk(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 6) throw std::runtime_error("topk expects 6 arguments");
  auto I = args[0].as_tensor();
  const int64_t k = args[1].as_int();
  const int64_t raw_direction = args[3].as_int();
  if (raw_direction != 0 && raw_direction != 1) throw std::runtime_error("Invalid enumeration value in operation arguments");
  const auto direction = static_cast<SortDirection>(raw_direction);
  const auto sort_type = validate<plaidml::op::TopKSortType>(args[4].as_int());
  const int64_t axis = static_cast<int64_t>(normalize_axis(args[2].as_int(), I.rank(), "topk"));
  Tensor order = argsort(I, static_cast<int>(axis), direction);
  Tensor first_k = index({TensorDim(k)}, 0);
  Tensor idxs_topk = gather(order, first_k).axis(axis);
  std::vector<Value> out;
  if (sort_type == plaidml::op::TopKSortType::VALUE) {
    Tensor values = sorted_by(I, order, axis);
    Tensor vals_topk = gather(values, first_k).axis(axis);
    out = {Value{vals_topk}, Value{idxs_topk}};
  } else {
    Tensor by_position = sorted_by(idxs_topk, argsort(idxs_topk, static_cast<int>(axis), SortDirection::ASC), axis);
    out = {Value{sorted_by(I, by_position, axis)}, Value{by_position}};
  }
  return Value(out);
}

// ---- non-maximum suppression (plaidml/op/lib/ops.cc:2034-2417) ------------------------------------------
using plaidml::op::BoxesDecodeMode;
using plaidml::op::NmsStyle;

Tensor larger_of(const Tensor& a, const Tensor& b) { return op_maximum(make_tuple(Value{a}, Value{b})).as_tensor(); }
Tensor smaller_of(const Tensor& a, const Tensor& b) { return op_minimum(make_tuple(Value{a}, Value{b})).as_tensor(); }
Tensor unit_clip(const Tensor& t) {
  return op_clip(make_tuple(Value{t}, Value{cast(Tensor(0.0), DType::FLOAT32)}, Value{cast(Tensor(1.0), DType::FLOAT32)})).as_tensor();
}
Tensor squeeze_at(const Tensor& t, int64_t axis) { return op_squeeze(make_tuple(Value{t}, int_tuple({axis}))).as_tensor(); }

// The four edges {y1, x1, y2, x2} of every box, each shaped like `boxes` with a last dimension of 1
// (ops.cc:2034-2117).  NMS boxes are corners in either order or centre + size; SSD boxes are priors in pixels that
// the location deltas, scaled by the variances, move and stretch.
std::vector<Tensor> box_edges(Tensor boxes, const Tensor& variances, const Tensor& location, BoxesDecodeMode decode, int64_t in_h,
                              int64_t in_w, bool clip_boxes, bool centered) {
  auto col = [](const Tensor& t, int k) -> Tensor { return gather(t, k).axis(3); };
  Tensor y1, x1, y2, x2;
  if (centered) {
    Tensor xc, yc, half_w, half_h;
    if (decode == BoxesDecodeMode::NMS) {
      xc = col(boxes, 0);
      yc = col(boxes, 1);
      half_w = col(boxes, 2) / 2.0;
      half_h = col(boxes, 3) / 2.0;
    } else if (decode == BoxesDecodeMode::SSD) {
      Tensor px1 = col(boxes, 0) / in_w, py1 = col(boxes, 1) / in_h, px2 = col(boxes, 2) / in_w, py2 = col(boxes, 3) / in_h;
      Tensor pw = px2 - px1, ph = py2 - py1;
      xc = col(variances, 0) * col(location, 0) * pw + (px1 + px2) / 2.0;
      yc = col(variances, 1) * col(location, 1) * ph + (py1 + py2) / 2.0;
      half_w = exp(col(variances, 2) * col(location, 2)) * pw / 2.0;
      half_h = exp(col(variances, 3) * col(location, 3)) * ph / 2.0;
    } else {
      throw std::runtime_error("Unrecognized boxes decode mode");
    }
    x1 = xc - half_w, x2 = xc + half_w, y1 = yc - half_h, y2 = yc + half_h;
  } else if (decode == BoxesDecodeMode::NMS) {
    Tensor ya = col(boxes, 0), xa = col(boxes, 1), yb = col(boxes, 2), xb = col(boxes, 3);
    y1 = smaller_of(ya, yb), x1 = smaller_of(xa, xb), y2 = larger_of(ya, yb), x2 = larger_of(xa, xb);
  } else if (decode == BoxesDecodeMode::SSD) {
    boxes = boxes / in_w + variances * location;
    x1 = col(boxes, 0), y1 = col(boxes, 1), x2 = col(boxes, 2), y2 = col(boxes, 3);
  } else {
    throw std::runtime_error("Unrecognized boxes decode mode");
  }
  if (clip_boxes) y1 = unit_clip(y1), x1 = unit_clip(x1), y2 = unit_clip(y2), x2 = unit_clip(x2);
  return {y1, x1, y2, x2};
}

// intersection over union of every pair of boxes: [batch, location class, box, box]; 0 where the union is empty
Tensor pairwise_iou(const std::vector<Tensor>& edges, const TensorDim& nb, const TensorDim& nbox, const TensorDim& nloc) {
  TensorDim one(1);
  Tensor zero = cast(index({one}, 0), edges[0].dtype());
  auto flat = [&](const Tensor& t) { return reshape(t, {nb, nloc, nbox}); };
  Tensor y1 = flat(edges[0]), x1 = flat(edges[1]), y2 = flat(edges[2]), x2 = flat(edges[3]);
  Tensor area = (y2 - y1) * (x2 - x1);
  auto rows = [&](const Tensor& t) { return reshape(t, {nb, nloc, nbox, one}); };
  auto cols = [&](const Tensor& t) { return reshape(t, {nb, nloc, one, nbox}); };
  Tensor ygap = smaller_of(rows(y2), cols(y2)) - larger_of(rows(y1), cols(y1));
  Tensor xgap = smaller_of(rows(x2), cols(x2)) - larger_of(rows(x1), cols(x1));
  Tensor inter = select(ygap > 0.0, ygap, zero) * select(xgap > 0.0, xgap, zero);
  Tensor uni = unsqueeze_at(area, -1) + unsqueeze_at(area, -2) - inter;
  return inter * select(uni <= 0.0, zero, 1.0 / uni);
}

// Greedy suppression unrolled max_output_boxes_per_class times over Scores [batch, class, box]: each round takes
// every (batch, class)'s best remaining box, records it, and zeroes the scores of the boxes overlapping it.
// Returns {selected (batch, class, box) triples, (batch, class, score) triples, number of valid selections};
// unused rows hold -1.
Value op_nms(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 21) throw std::runtime_error("nms expects 21 arguments");
  auto Boxes = args[0].as_tensor();
  auto Scores = args[1].as_tensor();
  auto iou_threshold = args[2].as_tensor();
  auto score_threshold = args[3].as_tensor();
  const int64_t max_per_class = args[4].as_int();
  const double sigma = args[5].as_float();
  const bool centered = args[6].as_bool();
  const bool sort_descending = args[7].as_bool();
  const auto out_type = validate<DType>(args[8].as_int());
  const auto decode = validate<BoxesDecodeMode>(args[9].as_int());
  const bool clip_before = args[10].as_bool(), clip_after = args[11].as_bool();
  const int64_t in_h = args[12].as_int(), in_w = args[13].as_int();
  const DType in_type = Boxes.dtype(), thr_type = iou_threshold.dtype();
  Tensor variances, location, arm_location;
  if (decode == BoxesDecodeMode::SSD) variances = args[14].as_tensor(), location = args[15].as_tensor();
  const bool with_arm = args[16].as_bool();
  if (with_arm) arm_location = args[17].as_tensor();
  const auto style = validate<NmsStyle>(args[18].as_int());
  const bool share_location = args[19].as_bool();
  const bool hard = args[20].as_bool();

  const int64_t boxes_count = Scores.compute_shape().sizes().at(2);
  std::vector<TensorDim> sd(Scores.rank());
  Scores.bind_dims(sd);
  TensorDim nb = sd[0], nc = sd[1], nbox = sd[2], one_dim(1);
  TensorDim nloc = share_location ? one_dim : nc;

  Tensor zero = cast(index({one_dim}, 0), in_type);
  Tensor zero_int = cast(zero, DType::INT32);
  Tensor one = zero + 1;
  Tensor neg1 = -one;
  Tensor neg1_out = cast(neg1, out_type);
  Tensor valid_outputs = zero;

  Boxes = unsqueeze_at(Boxes, 1);
  std::vector<Tensor> edges;
  if (with_arm) {
    variances = unsqueeze_at(variances, 1);
    auto p = box_edges(Boxes, variances, arm_location, decode, in_h, in_w, clip_before, centered);
    Tensor priors = concatenate({p[1], p[0], p[3], p[2]}, -1);
    edges = box_edges(priors, variances, location, decode, in_h, in_w, clip_before, centered);
  } else {
    if (decode == BoxesDecodeMode::SSD) variances = unsqueeze_at(variances, 1);
    edges = box_edges(Boxes, variances, location, decode, in_h, in_w, clip_before, centered);
  }
  Tensor iou = pairwise_iou(edges, nb, nbox, nloc);
  const double weight = sigma != 0 ? -0.5 / static_cast<float>(sigma) : 0.0;

  const float minus_ones[2] = {-1.f, -1.f};
  Buffer invalid_buf(TensorShape(DType::FLOAT32, {1, 1, 2}));
  invalid_buf.copy_from(minus_ones);
  Tensor invalid_node = cast(Constant(invalid_buf, "invalid_node"), out_type);

  const int64_t per_class = max_per_class != 0 ? std::min(boxes_count, max_per_class) : boxes_count;
  Tensor index_bc = cast(concatenate({index({nb, nc, one_dim}, 0), index({nb, nc, one_dim}, 1)}, 2), out_type);
  Tensor score_thr = cast(score_threshold, in_type);
  Tensor iou_thr = cast(iou_threshold, in_type);
  Tensor new_scores = select(Scores > score_thr, Scores, zero);

  auto zeros = [&](const std::vector<TensorDim>& dims) -> Tensor {
    std::vector<TensorIndex> idxs(3);
    return Contraction(dims, idxs, "nms").assign(zero(0));
  };
  auto top_k = [](const Tensor& t, int64_t k, int64_t axis, plaidml::op::TopKSortType type) {
    return op_topk(make_tuple(Value{t}, Value{k}, Value{axis}, Value{static_cast<int64_t>(SortDirection::DESC)},
                              Value{static_cast<int64_t>(type)}, Value{static_cast<int64_t>(DType::INT32)}))
        .as_tuple();
  };
  auto gather_nd = [](const Tensor& t, const Tensor& at, int64_t batch_dims) {
    return gatherBuilder(t, at, static_cast<uint64_t>(batch_dims), InterpolationMode::NONE).build();
  };
  auto sorted_desc = [](const Tensor& t, int64_t axis) { return sorted_by(t, argsort(t, static_cast<int>(axis), SortDirection::DESC), axis); };

  if (style == NmsStyle::CAFFE) {
    // only the top scores of each class take part
    auto top = top_k(new_scores, per_class, 2, plaidml::op::TopKSortType::VALUE);
    new_scores = scatter(zeros({nb, nc, nbox}), top[1].as_tensor(), top[0].as_tensor()).axis(2).mode(ScatterMode::UPDATE_ELT);
  } else if (style == NmsStyle::MXNET) {
    // every box competes in its best class only, and only the top boxes of a batch do
    Tensor best_class = squeeze_at(gather(argsort(new_scores, 1, SortDirection::DESC), 0).axis(1), 1);
    Tensor best_score = squeeze_at(gather(sorted_desc(new_scores, 1), 0).axis(1), 1);
    auto top = top_k(best_score, per_class, 1, plaidml::op::TopKSortType::INDEX);
    Tensor top_scores = top[0].as_tensor(), top_boxes = top[1].as_tensor();
    Tensor top_classes = gather_nd(best_class, unsqueeze_at(top_boxes, -1), 1);
    std::vector<TensorDim> dims(2);
    top_classes.bind_dims(dims);
    Tensor where = concatenate({unsqueeze_at(index(dims, 0), -1), unsqueeze_at(top_classes, -1), unsqueeze_at(top_boxes, -1)}, -1);
    new_scores = scatter(zeros({nb, nc, nbox}), where, top_scores).mode(ScatterMode::UPDATE_ND);
  }

  Tensor zero_cell = zeros({nb, nc, one_dim});
  std::vector<Tensor> box_parts, score_parts;
  for (int64_t k = 0; k < per_class; ++k) {
    Tensor candidate = gather(argsort(new_scores, 2, SortDirection::DESC), 0).axis(2);
    Tensor score = reshape(reduce(make_tuple(Value{new_scores}, Value{int64_t{2}}, Value{false}), "max", PLAIDML_AGG_OP_MAX).as_tensor(),
                           {nb, nc, one_dim});
    Tensor node = select(score > 0.0, index_bc, invalid_node);
    Tensor counted = reduce(make_tuple(Value{select(score != 0.0, one, zero)}, Value(), Value{false}), "sum", PLAIDML_AGG_OP_SUM).as_tensor();
    valid_outputs = valid_outputs + counted;
    score_parts.push_back(cast(node, thr_type));
    score = select(score > 0.0, score, neg1);
    score_parts.push_back(cast(score, thr_type));
    // the winner itself goes to zero by position (equal scores may exist), its neighbours by overlap
    Tensor cleared = scatter(new_scores, candidate, zero_cell).axis(2).mode(ScatterMode::UPDATE_ELT);
    new_scores = reshape(cleared, {nb, nc, nbox});
    Tensor class_idx;
    if (share_location) {
      class_idx = op_broadcast(make_tuple(Value{zero_int}, int_tuple(candidate.compute_shape().sizes()), int_tuple({1}))).as_tensor();
    } else {
      std::vector<TensorDim> cd(candidate.rank());
      candidate.bind_dims(cd);
      class_idx = index(cd, 1);
    }
    Tensor overlap = gather_nd(iou, concatenate({class_idx, candidate}, 2), 1);
    new_scores = select(hard ? overlap >= iou_thr : overlap > iou_thr, zero, new_scores);
    Tensor box_index = select(score > 0.0, cast(candidate, out_type), neg1_out);
    box_parts.push_back(node);
    box_parts.push_back(reshape(box_index, {nb, nc, one_dim}));
    if (sigma != 0) {
      new_scores = new_scores * exp(overlap * overlap * weight);
      new_scores = select(new_scores > score_thr, new_scores, zero);
    }
  }

  valid_outputs = cast(valid_outputs, out_type);
  TensorDim rows = nb * nc * per_class;
  Tensor scores_result = reshape(concatenate(score_parts, 2), {rows, TensorDim(3)});
  Tensor boxes_result = reshape(concatenate(box_parts, 2), {rows, TensorDim(3)});
  if (sort_descending) {
    Tensor key = reshape(gather(scores_result, 2).axis(1), {rows});
    Tensor order = argsort(key, 0, SortDirection::DESC);
    scores_result = gather(scores_result, order).axis(0);
    boxes_result = gather(boxes_result, order).axis(0);
  } else {
    // a stable sort on "own position, or past-the-end for a -1" moves the unused entries to the back
    TensorDim n = rows * 3;
    Tensor flat_scores = reshape(scores_result, {n}), flat_boxes = reshape(boxes_result, {n});
    Tensor key = select(flat_scores != cast(Tensor(-1), thr_type), index({n}, 0), cast(Tensor{n}, DType::INT32));
    Tensor order = argsort(cast(key, DType::FLOAT32), 0);
    scores_result = reshape(gather(flat_scores, order).axis(0), {rows, TensorDim(3)});
    boxes_result = reshape(gather(flat_boxes, order).axis(0), {rows, TensorDim(3)});
    if (decode == BoxesDecodeMode::SSD) {
      Tensor decoded = concatenate({edges[1], edges[0], edges[3], edges[2]}, -1);
      if (clip_after) decoded = unit_clip(decoded);
      Tensor out_boxes;
      if (share_location) {
        Tensor pick = gather(boxes_result, concatenate({zero_int, zero_int + 2}, 0)).axis(1);
        out_boxes = gather_nd(squeeze_at(decoded, 0), pick, 0);
      } else {
        out_boxes = gather_nd(decoded, boxes_result, 0);
      }
      if (style == NmsStyle::MXNET) {
        Tensor classes = gather(boxes_result, 1).axis(1) - 1;  // drops the background class
        Tensor one_int = zero_int + 1;
        scores_result = scatter(scores_result, one_int, cast(classes, scores_result.dtype())).mode(ScatterMode::UPDATE_SLICE).axis(1);
        boxes_result = scatter(boxes_result, one_int, classes).mode(ScatterMode::UPDATE_SLICE).axis(1);
      }
      scores_result = concatenate({scores_result, out_boxes}, 1);
    }
  }
  return make_tuple(boxes_result, scores_result, valid_outputs);
}

// plaidml/op/lib/ops.cc:1822-1918: both spatial dimensions of an image grow by integer factors.  NEAREST repeats
// pixels; BILINEAR spreads every pixel with a (2f-1) x (2f-1) tent kernel, which aligns the corners to 0 and
// f * (dim - 1) and treats the outside as zero.
Value op_image_resize(const Value& value) {
  auto args = value.as_tuple();
  if (args.size() != 4) throw std::runtime_error("image_resize expects 4 arguments");
  auto I = args[0].as_tensor();
  const auto factors = args[1].as_int_tuple();
  const auto interp = validate<plaidml::op::InterpolationMode>(args[2].as_int());
  const auto layout = validate<TensorLayout>(args[3].as_int());
  for (int64_t f : factors)
    if (f <= 0) throw std::runtime_error("All scaling factors in image_resize must be positive (received " + std::to_string(f) + ")");
  const size_t ndims = I.rank();
  int64_t pre_axes;
  switch (layout) {
    case TensorLayout::NCX: pre_axes = 2; break;
    case TensorLayout::NXC: pre_axes = 1; break;
    default: throw std::runtime_error("Unable to apply image_resize to a tensor with this layout");
  }
  if (ndims != 4) throw std::runtime_error("Expected 2 spatial dims for resize_images, received " + std::to_string(static_cast<int64_t>(ndims) - 2));
  if (factors.size() != 2)
    throw std::runtime_error("Cannot resize a 2D image using " + std::to_string(factors.size()) + " spatial scaling factors");
  if (interp == plaidml::op::InterpolationMode::NEAREST) {
    Value R = op_repeat(make_tuple(args[0], Value{factors[0]}, Value{pre_axes}));
    return op_repeat(make_tuple(R, Value{factors[1]}, Value{pre_axes + 1}));
  }
  if (interp != plaidml::op::InterpolationMode::BILINEAR) throw std::runtime_error("Unrecognized InterpolationMode in image_resize");
  Tensor HCoeff = cast(Tensor(1.0 / factors[0]), DType::FLOAT32);
  Tensor WCoeff = cast(Tensor(1.0 / factors[1]), DType::FLOAT32);
  TensorDim HFactor(factors[0]), WFactor(factors[1]);
  TensorIndex j("j"), i("i"), y("y"), x("x");
  Tensor HCoeffVec = Contraction({HFactor}, {y}, "image_resize").assign(HCoeff());
  Tensor WCoeffVec = Contraction({WFactor}, {x}, "image_resize").assign(WCoeff());
  TensorDim HK_dim = 2 * HFactor - 1, WK_dim = 2 * WFactor - 1;
  Tensor HK = Contraction({HK_dim}, {y}, "image_resize").sum(HCoeffVec(j + y - HFactor + 1)).add_constraint(j < HFactor);
  Tensor WK = Contraction({WK_dim}, {x}, "image_resize").sum(WCoeffVec(i + x - WFactor + 1)).add_constraint(i < WFactor);
  Tensor K = Contraction({HK_dim, WK_dim}, {y, x}, "image_resize").assign(HK(y) * WK(x));
  std::vector<TensorDim> I_dims(ndims), O_dims;
  std::vector<TensorIndex> I_idxs(ndims), O_idxs;
  I.bind_dims(I_dims);
  for (int64_t ax = 0; ax < pre_axes; ++ax) {
    O_dims.push_back(I_dims[ax]);
    O_idxs.push_back(I_idxs[ax]);
  }
  O_dims.push_back(HFactor * I_dims[pre_axes]);
  O_dims.push_back(WFactor * I_dims[pre_axes + 1]);
  O_idxs.push_back(HFactor * I_idxs[pre_axes] + j - HFactor + 1);
  O_idxs.push_back(WFactor * I_idxs[pre_axes + 1] + i - WFactor + 1);
  for (size_t ax = pre_axes + 2; ax < ndims; ++ax) {
    O_dims.push_back(I_dims[ax]);
    O_idxs.push_back(I_idxs[ax]);
  }
  Tensor O = Contraction(O_dims, O_idxs, "image_resize").sum(I(I_idxs) * K(j, i));
  return Value{O};
}

using OpFn = std::function<Value(const Value&)>;
const std::map<std::string, OpFn>& registry() {
  static const std::map<std::string, OpFn> r = {
      {"abs", op_abs},
      {"all", op_all},
      {"any", op_any},
      {"argmax", op_argmax},
      {"binary_crossentropy", op_binary_crossentropy},
      {"broadcast", op_broadcast},
      {"clip", op_clip},
      {"concatenate", op_concatenate},
      {"convolution", op_convolution},
      {"cumprod", op_cumprod},
      {"cumsum", op_cumsum},
      {"dot", op_dot},
      {"elu", op_elu},
      {"explicit_padding", op_explicit_padding},
      {"flip", op_flip},
      {"gatherND", op_gatherND},
      {"hard_sigmoid", op_hard_sigmoid},
      {"image_resize", op_image_resize},
      {"l2norm", op_l2norm},
      {"lrn", op_lrn},
      {"max", [](const Value& v) { return reduce(v, "max", PLAIDML_AGG_OP_MAX); }},
      {"maximum", op_maximum},
      {"mean", [](const Value& v) { return reduce(v, "mean", PLAIDML_AGG_OP_SUM); }},
      {"min", [](const Value& v) { return reduce(v, "min", PLAIDML_AGG_OP_MIN); }},
      {"minimum", op_minimum},
      {"nms", op_nms},
      {"mvn", op_mvn},
      {"pool", op_pool},
      {"prod", op_prod},
      {"relu", op_relu},
      {"reorg_yolo", op_reorg_yolo},
      {"repeat", op_repeat},
      {"reshape", op_reshape},
      {"scale_gradient", op_scale_gradient},
      {"sigmoid", op_sigmoid},
      {"slice", op_slice},
      {"softmax", op_softmax},
      {"sort", op_sort},
      {"spatial_padding", op_spatial_padding},
      {"square", op_square},
      {"squeeze", op_squeeze},
      {"sum", [](const Value& v) { return reduce(v, "sum", PLAIDML_AGG_OP_SUM); }},
      {"tile", op_tile},
      {"topk", op_topk},
      {"transpose", op_transpose},
      {"unsqueeze", op_unsqueeze},
      {"variance", op_variance},
  };
  return r;
}

}  // namespace

extern "C" plaidml_value* plaidml_op_make(plaidml_error* err, const char* op_name, plaidml_value* value) {
  err->code = 0;
  err->msg = nullptr;
  try {
    auto it = registry().find(op_name ? op_name : "");
    if (it == registry().end()) throw std::runtime_error(std::string("Invalid op_name: ") + (op_name ? op_name : "(null)"));
    // the library functions work on the C++ wrappers; hand them an aliasing copy of the argument
    plaidml_error e2{0, nullptr};
    Value arg(plaidml_value_clone(&e2, value));
    Value ret = it->second(arg);
    return plaidml_value_clone(&e2, ret.as_ptr());
  } catch (const std::exception& ex) {
    err->code = 1;
    err->msg = new plaidml_string{ex.what()};
    return nullptr;
  }
}

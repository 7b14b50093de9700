// The operation library for C++: the subset of the reference's builders
// (plaidml/op/op.h:28-1003) that the contraction hot path uses -- convolution,
// pool, dot, relu, mean / sum / max / min reductions, softmax, argmax, clip,
// maximum, minimum -- with the same names, argument order and defaults.  Each
// call goes through plaidml_op_make and emits EDSL contractions / elementwise
// operations.
#pragma once

#include <string>
#include <vector>

#include "plaidml/edsl/edsl.h"
#include "plaidml/op/ffi.h"

namespace plaidml {
namespace op {

inline void init() {
  plaidml::init();
  plaidml::edsl::init();
}

namespace details {
inline edsl::Value op(const std::string& name, const edsl::Value& args) {
  return edsl::Value(ffi::call<plaidml_value*>(plaidml_op_make, name.c_str(), args.as_ptr()));
}
}  // namespace details

enum class AutoGroupMode { UNGROUPED, EXPLICIT, AUTO, DEPTHWISE, _LAST };
enum class AutoPadMode { EXPLICIT, SAME_LOWER, SAME_UPPER, VALID, _LAST };
enum class ConvDerivMode { NONE, DATA, FILTER, _LAST };
enum class GroupLayout { NONE, SEPARATE, IN_C, IN_K, _LAST };
enum class PoolMode { AVG, MAX, MIN, SUM, _LAST };
enum class TensorLayout { NXC, NCX, KCX, XCK, GKCX, XGCK, _LAST };
enum class PadMode { CONSTANT, EDGE, REFLECT, SYMMETRIC, _LAST };
enum class EpsMode { ADD, MAX, _LAST };
enum class TopKSortType { VALUE, INDEX, _LAST };
enum class BoxesDecodeMode { NMS, SSD, _LAST };
enum class NmsStyle { CAFFE, MXNET, OV, _LAST };
enum class InterpolationMode { NEAREST, BILINEAR, _LAST };
// reshape: take the dimension from the input / infer it from the element count
static const int AUTO_DIM_MATCH = 0;
static const int AUTO_DIM_FILL = -1;

// a list of integers accepted from vectors and brace lists of the usual integer types
struct Integers {
  Integers(const std::vector<int>& elts) : value(edsl::make_tuple(elts)) {}                       // NOLINT
  Integers(const std::vector<int64_t>& elts) : value(edsl::make_tuple(elts)) {}                   // NOLINT
  Integers(const std::vector<size_t>& elts)                                                        // NOLINT
      : value(edsl::make_tuple(std::vector<int64_t>(elts.begin(), elts.end()))) {}
  Integers(const std::initializer_list<int>& elts) : Integers(std::vector<int>(elts)) {}           // NOLINT
  Integers(const std::initializer_list<int64_t>& elts) : Integers(std::vector<int64_t>(elts)) {}   // NOLINT
  Integers(const std::initializer_list<size_t>& elts) : Integers(std::vector<size_t>(elts)) {}     // NOLINT
  edsl::Value value;
};

inline edsl::Tensor all(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("all", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}

inline edsl::Tensor any(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("any", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}

inline edsl::Tensor binary_crossentropy(const edsl::Tensor& I, const edsl::Tensor& O, double epsilon) {
  return details::op("binary_crossentropy", edsl::make_tuple(I, O, epsilon)).as_tensor();
}

inline edsl::Tensor broadcast(const edsl::Tensor& I, const std::vector<int64_t>& result_shape,
                              const std::vector<int64_t>& bcast_axes) {
  return details::op("broadcast", edsl::make_tuple(I, edsl::make_tuple(result_shape), edsl::make_tuple(bcast_axes))).as_tensor();
}

inline edsl::Tensor cumprod(const edsl::Tensor& I, int axis) { return details::op("cumprod", edsl::make_tuple(I, axis)).as_tensor(); }

inline edsl::Tensor image_resize(const edsl::Tensor& I, const std::vector<int>& factors, InterpolationMode interpolation,
                                 TensorLayout layout) {
  return details::op("image_resize", edsl::make_tuple(I, edsl::make_tuple(factors), static_cast<int>(interpolation),
                                                      static_cast<int>(layout))).as_tensor();
}

class l2norm {
 public:
  explicit l2norm(const edsl::Tensor& I, const std::vector<int64_t> axes) : I_(I), axes_(axes) {}
  l2norm& epsilon(float epsilon) { epsilon_ = epsilon; return *this; }
  l2norm& eps_mode(EpsMode eps_mode) { eps_mode_ = eps_mode; return *this; }
  operator edsl::Tensor() const {
    return details::op("l2norm", edsl::make_tuple(I_, edsl::make_tuple(axes_), epsilon_, static_cast<int>(eps_mode_))).as_tensor();
  }

 private:
  edsl::Tensor I_;
  std::vector<int64_t> axes_;
  double epsilon_ = 0;
  EpsMode eps_mode_ = EpsMode::ADD;
};

class lrn {
 public:
  explicit lrn(const edsl::Tensor& I, const std::vector<int64_t>& window_size) : I_(I), window_size_(window_size) {}
  lrn& alpha(double alpha) { alpha_ = alpha; return *this; }
  lrn& beta(double beta) { beta_ = beta; return *this; }
  lrn& epsilon(double epsilon) { epsilon_ = epsilon; return *this; }
  lrn& window_size(const std::vector<int64_t>& window_size) { window_size_ = window_size; return *this; }
  lrn& axes(const std::vector<int64_t>& axes) { axes_ = axes; return *this; }
  operator edsl::Tensor() const {
    auto args = edsl::make_tuple(I_, edsl::make_tuple(window_size_), edsl::make_tuple(axes_), alpha_, beta_, epsilon_);
    return details::op("lrn", args).as_tensor();
  }

 private:
  edsl::Tensor I_;
  std::vector<int64_t> window_size_;
  std::vector<int64_t> axes_ = {-1};
  double alpha_ = 1., beta_ = 1., epsilon_ = 1.e-5;
};

class mvn {
 public:
  explicit mvn(const edsl::Tensor& I) : I_(I), axes_(edsl::None()) {}
  mvn& axes(const std::vector<int64_t>& axes) {
    if (!across_channels_ || !layout_.empty()) throw std::runtime_error("When using layout and across_channels, axes may not be specified");
    axes_ = edsl::make_tuple(axes);
    return *this;
  }
  mvn& across_channels(bool flag) {
    if (!axes_.is_none()) throw std::runtime_error("May not specify both axes and across_channels for MVN");
    across_channels_ = flag;
    return *this;
  }
  mvn& normalize_variance(bool flag) { normalize_variance_ = flag; return *this; }
  mvn& epsilon(double value) { epsilon_ = value; return *this; }
  mvn& layout(const std::string& value) {
    if (!axes_.is_none()) throw std::runtime_error("May not specify both axes and layout for MVN");
    layout_ = value;
    return *this;
  }
  operator edsl::Tensor() const {
    return details::op("mvn", edsl::make_tuple(I_, axes_, normalize_variance_, epsilon_, across_channels_, layout_)).as_tensor();
  }

 private:
  edsl::Tensor I_;
  edsl::Value axes_;
  bool normalize_variance_ = true;
  double epsilon_ = 1e-9;
  bool across_channels_ = true;
  std::string layout_;
};

inline edsl::Tensor reorg_yolo(const edsl::Tensor& I, int stride, bool decrease, const std::string& layout = "NCHW") {
  return details::op("reorg_yolo", edsl::make_tuple(I, stride, decrease, layout)).as_tensor();
}

inline edsl::Tensor scale_gradient(const edsl::Tensor& I, double scale = -1.0) {
  return details::op("scale_gradient", edsl::make_tuple(I, scale)).as_tensor();
}

class slice {
 public:
  explicit slice(const edsl::Tensor& I) : I_(I) {}
  slice& add_dims(const std::vector<int>& dims) {
    for (auto dim : dims) dims_.emplace_back(dim);
    return *this;
  }
  slice& add_dim(int dim) { dims_.emplace_back(dim); return *this; }
  slice& add_dim(int start, int stop, int step = 1) { dims_.emplace_back(edsl::make_tuple(start, stop, step)); return *this; }
  slice& add_dim(edsl::Value start, edsl::Value stop, edsl::Value step = edsl::Value(1)) {
    dims_.emplace_back(edsl::make_tuple(start, stop, step));
    return *this;
  }
  operator edsl::Tensor() const { return details::op("slice", edsl::make_tuple(I_, dims_)).as_tensor(); }

 private:
  edsl::Tensor I_;
  std::vector<edsl::Value> dims_;
};

class gatherND {
 public:
  explicit gatherND(const edsl::Tensor& x, const edsl::Tensor& y) : x_(x), y_(y) {}
  gatherND& interpolationMode(edsl::InterpolationMode mode) { interpolation_mode_ = mode; return *this; }
  gatherND& batchDims(int batch_dims) { batch_dims_ = batch_dims; return *this; }
  operator edsl::Tensor() const {  // NOLINT
    return details::op("gatherND", edsl::make_tuple(x_, y_, batch_dims_, static_cast<int>(interpolation_mode_))).as_tensor();
  }

 private:
  edsl::Tensor x_, y_;
  int64_t batch_dims_ = 0;
  edsl::InterpolationMode interpolation_mode_ = edsl::InterpolationMode::NONE;
};

inline edsl::Tensor sort(const edsl::Tensor& I, int axis, edsl::SortDirection direction = edsl::SortDirection::ASC) {
  return details::op("sort", edsl::make_tuple(I, axis, static_cast<int>(direction))).as_tensor();
}

// Non-maximum suppression over Boxes [batch, box, 4] and Scores [batch, class, box].  Three styles: OV (every
// score takes part), CAFFE (only each class's top scores) and MXNET (every box in its best class only, top boxes of
// the batch).  build() returns {selected (batch, class, box) triples, (batch, class, score) triples, the number of
// valid selections}; rows not used hold -1.
class nms {
 public:
  explicit nms(edsl::Tensor Boxes, edsl::Tensor Scores, edsl::Tensor IOU_threshold, edsl::Tensor Score_threshold,
               int max_output_boxes_per_class)
      : Boxes_(Boxes), Scores_(Scores), IOU_threshold_(IOU_threshold), Score_threshold_(Score_threshold),
        max_output_boxes_per_class_(max_output_boxes_per_class) {}
  nms& soft_nms_sigma(float v) { soft_nms_sigma_ = v; return *this; }
  nms& center_point_box(bool v) { center_point_box_ = v; return *this; }
  nms& sort_result_descending(bool v) { sort_result_descending_ = v; return *this; }
  nms& box_output_type(DType v) { box_output_type_ = v; return *this; }
  nms& boxes_decode_mode(BoxesDecodeMode v) { boxes_decode_mode_ = v; return *this; }
  nms& clip_before_nms(bool v) { clip_before_nms_ = v; return *this; }
  nms& clip_after_nms(bool v) { clip_after_nms_ = v; return *this; }
  nms& ssd_input_height(int v) { ssd_input_height_ = v; return *this; }
  nms& ssd_input_width(int v) { ssd_input_width_ = v; return *this; }
  nms& ssd_variances(edsl::Tensor v) { ssd_variances_ = v; return *this; }
  nms& ssd_location(edsl::Tensor v) { ssd_location_ = v; return *this; }
  nms& ssd_arm_location(edsl::Tensor v) { ssd_arm_location_ = v; return *this; }
  nms& ssd_with_arm_loc(bool v) { ssd_with_arm_loc_ = v; return *this; }
  nms& nms_style(NmsStyle v) { nms_style_ = v; return *this; }
  nms& share_location(bool v) { share_location_ = v; return *this; }
  nms& hard_suppression(bool v) { hard_suppression_ = v; return *this; }
  std::vector<edsl::Tensor> build() {
    auto args = edsl::make_tuple(Boxes_, Scores_, IOU_threshold_, Score_threshold_, max_output_boxes_per_class_,
                                 static_cast<double>(soft_nms_sigma_), center_point_box_, sort_result_descending_,
                                 static_cast<int>(box_output_type_), static_cast<int>(boxes_decode_mode_), clip_before_nms_,
                                 clip_after_nms_, ssd_input_height_, ssd_input_width_, ssd_variances_, ssd_location_,
                                 ssd_with_arm_loc_, ssd_arm_location_, static_cast<int>(nms_style_), share_location_,
                                 hard_suppression_);
    auto R = details::op("nms", args).as_tuple();
    return {R[0].as_tensor(), R[1].as_tensor(), R[2].as_tensor()};
  }

 private:
  edsl::Tensor Boxes_, Scores_, IOU_threshold_, Score_threshold_;
  edsl::Tensor ssd_variances_, ssd_location_, ssd_arm_location_;  // unset: passed as none
  int max_output_boxes_per_class_;
  float soft_nms_sigma_ = 0.0f;
  bool center_point_box_ = false;
  bool sort_result_descending_ = false;
  DType box_output_type_ = DType::INT32;
  BoxesDecodeMode boxes_decode_mode_ = BoxesDecodeMode::NMS;
  bool clip_before_nms_ = false, clip_after_nms_ = false;
  int ssd_input_height_ = 0, ssd_input_width_ = 0;
  bool ssd_with_arm_loc_ = false;
  NmsStyle nms_style_ = NmsStyle::OV;
  bool share_location_ = true;
  bool hard_suppression_ = true;
};

class topk {
 public:
  explicit topk(edsl::Tensor I, int k) : I_(I), k_(k) {}
  topk& axis(int axis) { axis_ = axis; return *this; }
  topk& sort_direction(edsl::SortDirection sort_direction) { sort_direction_ = sort_direction; return *this; }
  topk& sort_type(TopKSortType sort_type) { sort_type_ = sort_type; return *this; }
  topk& index_element_type(DType index_element_type) { index_element_type_ = index_element_type; return *this; }
  // {values, positions}
  std::vector<edsl::Tensor> build() {
    auto args = edsl::make_tuple(I_, k_, axis_, static_cast<int>(sort_direction_), static_cast<int>(sort_type_),
                                 static_cast<int>(index_element_type_));
    auto R = details::op("topk", args).as_tuple();
    return {R[0].as_tensor(), R[1].as_tensor()};
  }

 private:
  edsl::Tensor I_;
  int k_;
  int axis_ = -1;
  edsl::SortDirection sort_direction_ = edsl::SortDirection::DESC;
  TopKSortType sort_type_ = TopKSortType::VALUE;
  DType index_element_type_ = DType::INT32;
};

inline edsl::Tensor argmax(const edsl::Tensor& I, const edsl::Value& axes = edsl::None()) {
  return details::op("argmax", edsl::make_tuple(I, axes)).as_tensor();
}

inline edsl::Tensor clip(const edsl::Tensor& I, const edsl::Tensor& min, const edsl::Tensor& max) {
  return details::op("clip", edsl::make_tuple(I, min, max)).as_tensor();
}

// NXC (x) XCK forward convolution; defaults: stride 1, no dilation, SAME_UPPER padding, ungrouped
class convolution {
 public:
  explicit convolution(edsl::Tensor I, edsl::Tensor F) : I_(I), F_(F) {}
  convolution& strides(Integers elts) { strides_ = elts.value; return *this; }
  convolution& dilations(Integers elts) { dilations_ = elts.value; return *this; }
  convolution& data_dilations(Integers elts) { data_dilations_ = elts.value; return *this; }
  convolution& filter_shape(Integers elts) { filter_shape_ = elts.value; return *this; }
  convolution& groups(int groups) { groups_ = groups; return *this; }
  convolution& manual_padding(Integers elts) { manual_padding_ = elts.value; return *this; }
  convolution& autopad_mode(AutoPadMode mode) { autopad_mode_ = mode; return *this; }
  convolution& input_layout(TensorLayout layout) { input_layout_ = layout; return *this; }
  convolution& filter_layout(TensorLayout layout) { filter_layout_ = layout; return *this; }
  convolution& group_layout(GroupLayout layout) { group_layout_ = layout; return *this; }
  convolution& winograd_allowed(bool allowed) { winograd_allowed_ = allowed; return *this; }
  convolution& name(const std::string& name) { name_ = name; return *this; }
  convolution& autogroup_mode(AutoGroupMode mode) { autogroup_mode_ = mode; return *this; }
  convolution& deriv_mode(ConvDerivMode mode) { deriv_mode_ = mode; return *this; }
  convolution& result_shape(Integers elts) { result_shape_ = elts.value; return *this; }
  convolution& infer_result_shape(bool infer) { infer_result_shape_ = infer; return *this; }

  operator edsl::Tensor() const {  // NOLINT
    auto args = edsl::make_tuple(I_, F_, strides_, dilations_, data_dilations_, filter_shape_, groups_,
                                 static_cast<int>(autopad_mode_), manual_padding_, static_cast<int>(input_layout_),
                                 static_cast<int>(filter_layout_), static_cast<int>(group_layout_), winograd_allowed_, name_,
                                 static_cast<int>(autogroup_mode_), static_cast<int>(deriv_mode_), result_shape_,
                                 infer_result_shape_);
    return details::op("convolution", args).as_tensor();
  }

 private:
  edsl::Tensor I_, F_;
  edsl::Value strides_, dilations_, data_dilations_, filter_shape_;
  int groups_ = 1;
  edsl::Value manual_padding_;
  AutoPadMode autopad_mode_ = AutoPadMode::SAME_UPPER;
  TensorLayout input_layout_ = TensorLayout::NXC;
  TensorLayout filter_layout_ = TensorLayout::XCK;
  GroupLayout group_layout_ = GroupLayout::NONE;
  bool winograd_allowed_ = false;
  std::string name_;
  AutoGroupMode autogroup_mode_ = AutoGroupMode::UNGROUPED;
  ConvDerivMode deriv_mode_ = ConvDerivMode::NONE;
  edsl::Value result_shape_;
  bool infer_result_shape_ = false;
};

inline edsl::Tensor abs(const edsl::Tensor& I) { return details::op("abs", edsl::make_tuple(I)).as_tensor(); }

inline edsl::Tensor concatenate(const std::vector<edsl::Tensor>& tensors, int axis) {
  return details::op("concatenate", edsl::make_tuple(edsl::make_tuple(tensors), axis)).as_tensor();
}

inline edsl::Tensor cumsum(const edsl::Tensor& I, int axis, bool exclusive = false) {
  return details::op("cumsum", edsl::make_tuple(I, axis, exclusive)).as_tensor();
}

inline edsl::Tensor elu(const edsl::Tensor& I, double alpha) { return details::op("elu", edsl::make_tuple(I, alpha)).as_tensor(); }

class explicit_padding {
 public:
  explicit explicit_padding(const edsl::Tensor& I, const std::vector<int>& lo_pads, const std::vector<int>& hi_pads)
      : I_(I), lo_pads_(lo_pads), hi_pads_(hi_pads), mode_(PadMode::CONSTANT), padval_(edsl::Constant(0)) {}
  explicit_padding& lo_pads(const std::vector<int>& lo_pads) { lo_pads_ = lo_pads; return *this; }
  explicit_padding& hi_pads(const std::vector<int>& hi_pads) { hi_pads_ = hi_pads; return *this; }
  explicit_padding& mode(PadMode mode) { mode_ = mode; return *this; }
  explicit_padding& padval(const edsl::Tensor& padval) { padval_ = padval; return *this; }
  operator edsl::Tensor() const {  // NOLINT
    auto args = edsl::make_tuple(I_, edsl::make_tuple(lo_pads_), edsl::make_tuple(hi_pads_), static_cast<int>(mode_), padval_);
    return details::op("explicit_padding", args).as_tensor();
  }

 private:
  edsl::Tensor I_;
  std::vector<int> lo_pads_, hi_pads_;
  PadMode mode_;
  edsl::Tensor padval_;
};

inline edsl::Tensor flip(const edsl::Tensor& I, int axis) { return details::op("flip", edsl::make_tuple(I, axis)).as_tensor(); }

inline edsl::Tensor hard_sigmoid(const edsl::Tensor& I, double slope) {
  return details::op("hard_sigmoid", edsl::make_tuple(I, slope)).as_tensor();
}

inline edsl::Tensor dot(const edsl::Tensor& I, const edsl::Tensor& K, const std::string& name = "") {
  return details::op("dot", edsl::make_tuple(I, K, name)).as_tensor();
}

inline edsl::Tensor max(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {  // NOLINT
  return details::op("max", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}
inline edsl::Tensor maximum(const edsl::Tensor& X, const edsl::Tensor& Y) {
  return details::op("maximum", edsl::make_tuple(X, Y)).as_tensor();
}
inline edsl::Tensor mean(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("mean", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}
inline edsl::Tensor min(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {  // NOLINT
  return details::op("min", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}
inline edsl::Tensor minimum(const edsl::Tensor& X, const edsl::Tensor& Y) {
  return details::op("minimum", edsl::make_tuple(X, Y)).as_tensor();
}

inline edsl::Tensor pool(const edsl::Tensor I, PoolMode pool_mode, const std::vector<int>& pool_size,
                         const std::vector<int>& strides, AutoPadMode autopad_mode, const std::vector<int>& manual_padding,
                         TensorLayout input_layout, bool include_padding_in_avg = false,
                         bool use_ceil_for_output_shape = false, const std::string& name = "") {
  auto args = edsl::make_tuple(I, static_cast<int>(pool_mode), edsl::make_tuple(pool_size), edsl::make_tuple(strides),
                               static_cast<int>(autopad_mode), edsl::make_tuple(manual_padding),
                               static_cast<int>(input_layout), include_padding_in_avg, use_ceil_for_output_shape, name);
  return details::op("pool", args).as_tensor();
}

inline edsl::Tensor prod(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("prod", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}

class relu {
 public:
  explicit relu(const edsl::Tensor& I) : I_(I) {}
  relu& alpha(const edsl::Tensor& alpha) { alpha_ = alpha; return *this; }
  relu& max_value(const edsl::Tensor& max_value) { max_value_ = max_value; return *this; }
  relu& threshold(double threshold) { threshold_ = edsl::Value(threshold); return *this; }
  relu& name(const std::string& name) { name_ = name; return *this; }
  operator edsl::Tensor() const {  // NOLINT
    return details::op("relu", edsl::make_tuple(I_, alpha_, max_value_, threshold_, name_)).as_tensor();
  }

 private:
  edsl::Tensor I_, alpha_, max_value_;
  edsl::Value threshold_;
  std::string name_;
};

inline edsl::Tensor repeat(const edsl::Tensor& I, int repeats, int axis) {
  return details::op("repeat", edsl::make_tuple(I, repeats, axis)).as_tensor();
}

inline edsl::Tensor reshape(const edsl::Tensor& I, const edsl::Value& dims) {
  return details::op("reshape", edsl::make_tuple(I, dims)).as_tensor();
}

inline edsl::Tensor sigmoid(const edsl::Tensor& I) { return details::op("sigmoid", edsl::make_tuple(I)).as_tensor(); }

inline edsl::Tensor spatial_padding(const edsl::Tensor& x, const std::vector<int>& lo_pads, const std::vector<int>& hi_pads,
                                    TensorLayout data_layout) {
  auto args = edsl::make_tuple(x, edsl::make_tuple(lo_pads), edsl::make_tuple(hi_pads), static_cast<int>(data_layout));
  return details::op("spatial_padding", args).as_tensor();
}

inline edsl::Tensor square(const edsl::Tensor& x) { return details::op("square", edsl::Value(x)).as_tensor(); }

inline edsl::Tensor squeeze(const edsl::Tensor& I, const std::vector<int>& axes) {
  return details::op("squeeze", edsl::make_tuple(I, edsl::make_tuple(axes))).as_tensor();
}

inline edsl::Tensor softmax(const edsl::Tensor& I, int axis, const std::string& name = "") {
  return details::op("softmax", edsl::make_tuple(I, axis, name)).as_tensor();
}

inline edsl::Tensor sum(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("sum", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}

inline edsl::Tensor tile(const edsl::Tensor& I, const std::vector<int>& tiling_factors) {
  return details::op("tile", edsl::make_tuple(I, edsl::make_tuple(tiling_factors))).as_tensor();
}

inline edsl::Tensor transpose(const edsl::Tensor& I, const edsl::Value& axes = edsl::None()) {
  return details::op("transpose", edsl::make_tuple(I, axes)).as_tensor();
}

inline edsl::Tensor unsqueeze(const edsl::Tensor& I, const std::vector<int64_t>& axes) {
  return details::op("unsqueeze", edsl::make_tuple(I, edsl::make_tuple(axes))).as_tensor();
}

inline edsl::Tensor variance(const edsl::Tensor& I, const edsl::Value& axes = edsl::None(), bool keepdims = false) {
  return details::op("variance", edsl::make_tuple(I, axes, keepdims)).as_tensor();
}

}  // namespace op
}  // namespace plaidml

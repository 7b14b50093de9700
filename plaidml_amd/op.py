"""Python view of the operation library (plaidml_op_make), after plaidml/op/__init__.py of the
reference.  Keyword defaults follow the C++ builders of plaidml/op/op.h."""
from . import edsl as E

# enumerations of plaidml/op/op.h:28-130
AUTOGROUP_UNGROUPED, AUTOGROUP_EXPLICIT, AUTOGROUP_AUTO, AUTOGROUP_DEPTHWISE = range(4)
AUTOPAD_EXPLICIT, AUTOPAD_SAME_LOWER, AUTOPAD_SAME_UPPER, AUTOPAD_VALID = range(4)
GROUP_NONE, GROUP_SEPARATE, GROUP_IN_C, GROUP_IN_K = range(4)
POOL_AVG, POOL_MAX, POOL_MIN, POOL_SUM = range(4)
LAYOUT_NXC, LAYOUT_NCX, LAYOUT_KCX, LAYOUT_XCK, LAYOUT_GKCX, LAYOUT_XGCK = range(6)

SAME_UPPER, SAME_LOWER, VALID, EXPLICIT = 'same_upper', 'same_lower', 'valid', 'explicit'
_AUTOPAD = {SAME_UPPER: AUTOPAD_SAME_UPPER, SAME_LOWER: AUTOPAD_SAME_LOWER, VALID: AUTOPAD_VALID, EXPLICIT: AUTOPAD_EXPLICIT}
_POOL = {'avg': POOL_AVG, 'max': POOL_MAX, 'min': POOL_MIN, 'sum': POOL_SUM}


def _ints(x):
    return None if x is None else [int(v) for v in x]


DERIV_NONE, DERIV_DATA, DERIV_FILTER = range(3)


def convolution(I, F, strides=None, dilations=None, data_dilations=None, autopad=SAME_UPPER, manual_padding=None,
                depthwise=False, name='', groups=1, input_layout=LAYOUT_NXC, filter_layout=LAYOUT_XCK,
                group_layout=GROUP_NONE, autogroup_mode=AUTOGROUP_UNGROUPED, deriv_mode=DERIV_NONE, result_shape=None,
                infer_result_shape=False, filter_shape=None):
    """The 18 arguments of the reference's convolution (plaidml/op/op.h:192-335).  With deriv_mode DATA the first
    tensor is the forward result, with FILTER the second one is.  depthwise=True is GroupLayout IN_C with
    AutoGroupMode DEPTHWISE."""
    if depthwise:
        group_layout, autogroup_mode = GROUP_IN_C, AUTOGROUP_DEPTHWISE
    args = [I, F, _ints(strides), _ints(dilations), _ints(data_dilations), _ints(filter_shape), int(groups), _AUTOPAD[autopad],
            _ints(manual_padding), int(input_layout), int(filter_layout), int(group_layout), False, name,
            int(autogroup_mode), int(deriv_mode), _ints(result_shape), bool(infer_result_shape)]
    return E.op_make('convolution', args).as_tensor()


def pool(I, mode, pool_size, strides, autopad=VALID, manual_padding=None, include_padding_in_avg=False, use_ceil=False,
         name=''):
    args = [I, _POOL[mode], _ints(pool_size), _ints(strides), _AUTOPAD[autopad], _ints(manual_padding or []), LAYOUT_NXC,
            bool(include_padding_in_avg), bool(use_ceil), name]
    return E.op_make('pool', args).as_tensor()


def dot(X, Y, name=''):
    return E.op_make('dot', [X, Y, name]).as_tensor()


def _axes(axes):
    if axes is None or isinstance(axes, int):
        return axes
    return [int(a) for a in axes]


def sum(I, axes=None, keepdims=False):  # noqa: A001
    return E.op_make('sum', [I, _axes(axes), bool(keepdims)]).as_tensor()


def max(I, axes=None, keepdims=False):  # noqa: A001
    return E.op_make('max', [I, _axes(axes), bool(keepdims)]).as_tensor()


def min(I, axes=None, keepdims=False):  # noqa: A001
    return E.op_make('min', [I, _axes(axes), bool(keepdims)]).as_tensor()


def mean(I, axes=None, keepdims=False):
    return E.op_make('mean', [I, _axes(axes), bool(keepdims)]).as_tensor()


def relu(I):
    return E.op_make('relu', [I, None, None, None, '']).as_tensor()


def softmax(I, axis=-1, name=''):
    return E.op_make('softmax', [I, int(axis), name]).as_tensor()


def argmax(I, axis=-1):
    return E.op_make('argmax', [I, _axes(axis)]).as_tensor()


def clip(I, lo, hi):
    return E.op_make('clip', [I, lo, hi]).as_tensor()


def maximum(X, Y):
    return E.op_make('maximum', [X, Y]).as_tensor()


def minimum(X, Y):
    return E.op_make('minimum', [X, Y]).as_tensor()


PAD_CONSTANT, PAD_EDGE, PAD_REFLECT, PAD_SYMMETRIC = range(4)
AUTO_DIM_MATCH, AUTO_DIM_FILL = 0, -1


def abs(I):  # noqa: A001
    return E.op_make('abs', [I]).as_tensor()


def concatenate(tensors, axis):
    return E.op_make('concatenate', [list(tensors), int(axis)]).as_tensor()


def cumsum(I, axis, exclusive=False):
    return E.op_make('cumsum', [I, int(axis), bool(exclusive)]).as_tensor()


def elu(I, alpha):
    return E.op_make('elu', [I, alpha]).as_tensor()


def explicit_padding(I, lo_pads, hi_pads, mode=PAD_CONSTANT, padval=0):
    pv = padval if isinstance(padval, E.Tensor) else E.Constant(padval)
    return E.op_make('explicit_padding', [I, _ints(lo_pads), _ints(hi_pads), int(mode), pv]).as_tensor()


def flip(I, axis=None):
    return E.op_make('flip', [I, _axes(axis)]).as_tensor()


def hard_sigmoid(I, slope):
    return E.op_make('hard_sigmoid', [I, float(slope)]).as_tensor()


def prod(I, axes=None, keepdims=False):
    return E.op_make('prod', [I, _axes(axes), bool(keepdims)]).as_tensor()


def repeat(I, repeats, axis):
    return E.op_make('repeat', [I, int(repeats), int(axis)]).as_tensor()


def reshape(I, dims):
    return E.op_make('reshape', [I, [None if d is None else int(d) for d in dims]]).as_tensor()


def sigmoid(I):
    return E.op_make('sigmoid', [I]).as_tensor()


def spatial_padding(I, lo_pads, hi_pads, layout=LAYOUT_NXC):
    return E.op_make('spatial_padding', [I, _ints(lo_pads), _ints(hi_pads), int(layout)]).as_tensor()


def square(I):
    return E.op_make('square', [I]).as_tensor()


def squeeze(I, axes):
    return E.op_make('squeeze', [I, _axes(axes)]).as_tensor()


def tile(I, tiling_factors):
    return E.op_make('tile', [I, _ints(tiling_factors)]).as_tensor()


def transpose(I, axes=None):
    return E.op_make('transpose', [I, _axes(axes)]).as_tensor()


def unsqueeze(I, axes):
    return E.op_make('unsqueeze', [I, _axes(axes)]).as_tensor()


def variance(I, axes=None, keepdims=False):
    return E.op_make('variance', [I, _axes(axes), bool(keepdims)]).as_tensor()


EPS_ADD, EPS_MAX = range(2)


def all(I, axes=None, keepdims=False):  # noqa: A001
    return E.op_make('all', [I, _axes(axes), bool(keepdims)]).as_tensor()


def any(I, axes=None, keepdims=False):  # noqa: A001
    return E.op_make('any', [I, _axes(axes), bool(keepdims)]).as_tensor()


def binary_crossentropy(targets, preds, epsilon):
    return E.op_make('binary_crossentropy', [targets, preds, float(epsilon)]).as_tensor()


def broadcast(I, result_shape, bcast_axes):
    return E.op_make('broadcast', [I, _ints(result_shape), _ints(bcast_axes)]).as_tensor()


def cumprod(I, axis):
    return E.op_make('cumprod', [I, int(axis)]).as_tensor()


def l2norm(I, axes, epsilon=0.0, eps_mode=EPS_ADD):
    return E.op_make('l2norm', [I, _ints(axes), float(epsilon), int(eps_mode)]).as_tensor()


def lrn(I, window_size, axes=(-1,), alpha=1.0, beta=1.0, epsilon=1e-5):
    return E.op_make('lrn', [I, _ints(window_size), _ints(axes), float(alpha), float(beta), float(epsilon)]).as_tensor()


def mvn(I, axes=None, normalize_variance=True, epsilon=1e-9, across_channels=True, layout=''):
    return E.op_make('mvn', [I, _axes(axes), bool(normalize_variance), float(epsilon), bool(across_channels), layout]).as_tensor()


def reorg_yolo(I, stride, decrease, layout='NCHW'):
    return E.op_make('reorg_yolo', [I, int(stride), bool(decrease), layout]).as_tensor()


def scale_gradient(I, scale=-1.0):
    return E.op_make('scale_gradient', [I, float(scale)]).as_tensor()


def slice_of(I, slices):
    """Each entry an int or a Python slice, as plaidml/op/__init__.py:246-257."""
    out = []
    for s in slices:
        if isinstance(s, int):
            out.append(s)
        elif isinstance(s, slice):
            out.append([s.start, s.stop, s.step])
        else:
            raise ValueError('Unexpected type {} used to slice tensor'.format(type(s)))
    return E.op_make('slice', [I, out]).as_tensor()


TOPK_VALUE, TOPK_INDEX = range(2)


def gatherND(x, y, batch_dims=0, interpolation_mode=E.INTERP_NONE):
    return E.op_make('gatherND', [x, y, int(batch_dims), int(interpolation_mode)]).as_tensor()


def sort(I, axis=-1, direction=E.SORT_ASC):
    return E.op_make('sort', [I, int(axis), int(direction)]).as_tensor()


def topk(I, k, axis=-1, sort_direction=E.SORT_DESC, sort_type=TOPK_VALUE, index_element_type=E.DType.INT32):
    """Returns (values, positions)."""
    r = E.op_make('topk', [I, int(k), int(axis), int(sort_direction), int(sort_type), int(index_element_type)]).as_tuple()
    return r[0].as_tensor(), r[1].as_tensor()


BOXES_NMS, BOXES_SSD = range(2)
NMS_CAFFE, NMS_MXNET, NMS_OV = range(3)


def nms(Boxes, Scores, iou_threshold, score_threshold, max_output_boxes_per_class, soft_nms_sigma=0.0,
        center_point_box=False, sort_result_descending=False, box_output_type=E.DType.INT32,
        boxes_decode_mode=BOXES_NMS, clip_before_nms=False, clip_after_nms=False, ssd_input_height=0,
        ssd_input_width=0, ssd_variances=None, ssd_location=None, ssd_with_arm_loc=False, ssd_arm_location=None,
        nms_style=NMS_OV, share_location=True, hard_suppression=True):
    """Non-maximum suppression; the arguments and defaults of the C++ builder plaidml::op::nms.  Returns
    [selected (batch, class, box) triples, (batch, class, score) triples, number of valid selections]."""
    r = E.op_make('nms', [Boxes, Scores, iou_threshold, score_threshold, int(max_output_boxes_per_class),
                          float(soft_nms_sigma), bool(center_point_box), bool(sort_result_descending),
                          int(box_output_type), int(boxes_decode_mode), bool(clip_before_nms), bool(clip_after_nms),
                          int(ssd_input_height), int(ssd_input_width), ssd_variances, ssd_location,
                          bool(ssd_with_arm_loc), ssd_arm_location, int(nms_style), bool(share_location),
                          bool(hard_suppression)]).as_tuple()
    return [v.as_tensor() for v in r]


RESIZE_NEAREST, RESIZE_BILINEAR = range(2)


def image_resize(I, factors, interp=RESIZE_NEAREST, layout=LAYOUT_NXC):
    return E.op_make('image_resize', [I, _ints(factors), int(interp), int(layout)]).as_tensor()

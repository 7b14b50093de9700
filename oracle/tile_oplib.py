"""Op-library subset of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Restates, on top of oracle/tile_oracle.py, the contractions that the reference
op library emits for the operations on the hot path (plaidml/op/lib/ops.cc):

  convolution   :879-1467 with the validation of :671-877 (NXC / NCX data, XCK / KCX /
                 XGCK / GKCX filters; strides, dilations, data dilations, autopad,
                 explicit padding; the four group layouts and autogroup modes; the
                 DATA and FILTER derivative modes), padding rules :347-418
  pool          :2562-2703 (MAX / MIN / SUM / AVG, NXC)
  dot           :1512-1561
  mean          :1970-2003, sum / max via the same AggregationAxes :71-127
  relu          :2705-2728 (plain form only)
  softmax       :3049-3098 (last-axis form)
  argmax        :505-521
  and, each cited where it is defined below: abs, all, any, binary_crossentropy,
  broadcast, clip, concatenate, cumprod, cumsum, elu, explicit_padding, flip,
  gatherND, hard_sigmoid, image_resize, l2norm, lrn, mvn, nms, prod, reorg_yolo, repeat,
  reshape, scale_gradient, sigmoid, slice, sort, spatial_padding, square, squeeze,
  tile, topk, transpose, unsqueeze, variance

Pinned by tests/test_oplib_ops.py, tests/test_conv_general.py and the op-level
cases of tests/test_oracle_golden.py (numpy closed forms, the exact cases of
plaidml/op/op_test.cc, direct numpy evaluations of the definitions).
nms has no test in the reference: tests/test_nms.py pins it against a loop-written
greedy suppression for the NMS box formats and the three styles, its SSD box
decoding (_box_corners) against boxes worked out by hand from ops.cc:2034-2117 and the
box columns of whole SSD results against a box-by-box scalar decoding.

Nothing in the shipped package imports this module.
"""
import builtins

import numpy as np

from . import tile_oracle as E

SAME_UPPER, SAME_LOWER, VALID, EXPLICIT = 'same_upper', 'same_lower', 'valid', 'explicit'


def compute_padding_and_output_size(input_size, filter_size, stride, autopad, pad_lo=0, pad_hi=0,
                                    dilation=1, data_dilation=1, use_ceil=False):
    """plaidml/op/lib/ops.cc:347-382.  Integer division is C division of non-negative values."""
    i_eff = data_dilation * (input_size - 1) + 1
    f_eff = dilation * (filter_size - 1) + 1
    ceil_term = stride - 1 if use_ceil else 0
    if autopad == EXPLICIT:
        return pad_lo, (i_eff + pad_lo + pad_hi - f_eff + stride + ceil_term) // stride
    if autopad == VALID:
        return 0, (i_eff - f_eff + stride + ceil_term) // stride
    if autopad in (SAME_LOWER, SAME_UPPER):
        out = (i_eff + stride - 1) // stride
        lower = 1 if autopad == SAME_LOWER else 0
        pad = (builtins.max(0, (out - 1) * stride + f_eff - i_eff) + lower) // 2
        return pad, out
    raise ValueError('Unexpected autopadding mode: %s' % autopad)


def compute_padding_and_input_size(output_size, filter_size, stride, autopad, pad_lo=0, pad_hi=0, dilation=1,
                                   data_dilation=1):
    """plaidml/op/lib/ops.cc:383-418: the smallest input extent giving `output_size`.  The SAME modes return the
    output extent itself as the input extent (so written there)."""
    if data_dilation != 1:
        raise ValueError('Cannot infer input data size for transposed convolution with data dilation')
    f_eff = dilation * (filter_size - 1) + 1
    if autopad == EXPLICIT:
        return pad_lo, output_size * stride - pad_lo - pad_hi + f_eff - stride
    if autopad == VALID:
        return 0, output_size * stride + f_eff - stride
    if autopad in (SAME_LOWER, SAME_UPPER):
        input_size = output_size * stride - stride + 1
        lower = 1 if autopad == SAME_LOWER else 0
        return (builtins.max(0, (output_size - 1) * stride + f_eff - input_size) + lower) // 2, output_size
    raise ValueError('Unexpected autopadding mode: %s' % autopad)


LAYOUT_NXC, LAYOUT_NCX, LAYOUT_KCX, LAYOUT_XCK, LAYOUT_GKCX, LAYOUT_XGCK = range(6)
GROUP_NONE, GROUP_SEPARATE, GROUP_IN_C, GROUP_IN_K = range(4)
AUTOGROUP_UNGROUPED, AUTOGROUP_EXPLICIT, AUTOGROUP_AUTO, AUTOGROUP_DEPTHWISE = range(4)
DERIV_NONE, DERIV_DATA, DERIV_FILTER = range(3)


def _data_order(layout, n, c, spatial):
    return [n] + ([c] if layout == LAYOUT_NCX else []) + list(spatial) + ([c] if layout == LAYOUT_NXC else [])


def _filter_order(layout, g, k, c, spatial):
    if layout in (LAYOUT_GKCX, LAYOUT_KCX):
        return ([g] if layout == LAYOUT_GKCX else []) + [k, c] + list(spatial)
    return list(spatial) + ([g] if layout == LAYOUT_XGCK else []) + [c, k]


def convolution(I_or_O, F_or_O, strides=None, dilations=None, data_dilations=None, autopad=SAME_UPPER,
                manual_padding=None, depthwise=False, name='conv', groups=1, input_layout=LAYOUT_NXC,
                filter_layout=LAYOUT_XCK, group_layout=GROUP_NONE, autogroup_mode=AUTOGROUP_UNGROUPED,
                deriv_mode=DERIV_NONE, result_shape=None, infer_result_shape=False, filter_shape=None):
    """plaidml/op/lib/ops.cc:879-1467 with the validation of :671-877, on concrete shapes.  One contraction over
    I (data), F (filters), O (forward result); deriv_mode names the one computed: NONE -> O, DATA -> I (first
    argument is O), FILTER -> F (second argument is O).  depthwise=True is the IN_C layout with DEPTHWISE grouping."""
    if depthwise:
        group_layout, autogroup_mode = GROUP_IN_C, AUTOGROUP_DEPTHWISE
    if input_layout not in (LAYOUT_NXC, LAYOUT_NCX):
        raise ValueError('Input tensor layout requested in conv op does not apply to convolution input tensors')
    if filter_layout not in (LAYOUT_KCX, LAYOUT_XCK, LAYOUT_GKCX, LAYOUT_XGCK):
        raise ValueError('Filter tensor layout requested in conv op does not apply to convolution filter tensors')
    separate = filter_layout in (LAYOUT_GKCX, LAYOUT_XGCK)
    rank = len(strides) if strides else len(I_or_O.shape) - 2
    strides = list(strides or [1] * rank)
    dilations = list(dilations or [1] * rank)
    data_dilations = list(data_dilations or [1] * rank)
    manual_padding = list(manual_padding or [])
    result_shape = list(result_shape or [])
    if manual_padding and autopad != EXPLICIT:
        raise ValueError('Autopadding and manual padding both requested for single conv operation')
    if len(dilations) != rank or len(data_dilations) != rank:
        raise ValueError('Inconsistent spatial rank in conv op')
    if separate != (group_layout == GROUP_SEPARATE):
        raise ValueError('Filter layout and group layout disagree about separate groups')
    if not result_shape and deriv_mode != DERIV_NONE and not infer_result_shape:
        raise ValueError('Transposed/gradient convolutions require specifying the result_shape')
    if result_shape and len(result_shape) != rank:
        raise ValueError('Inconsistent spatial rank in conv op (result shape)')
    while len(manual_padding) < rank:
        manual_padding.append(0)
    while len(manual_padding) < 2 * rank:
        manual_padding.append(manual_padding[len(manual_padding) - rank])  # pad_hi defaults to pad_lo
    # grouping strategy, ops.cc:811-875
    if autogroup_mode == AUTOGROUP_UNGROUPED:
        if groups != 1:
            raise ValueError('Convolution AutoGroupMode::UNGROUPED requires groups == 1')
    elif autogroup_mode == AUTOGROUP_AUTO:
        if group_layout == GROUP_NONE:
            groups, autogroup_mode = 1, AUTOGROUP_UNGROUPED
        if group_layout == GROUP_IN_C:
            raise ValueError('Cannot automatically detect group size of convolution with IN_C GroupLayout')
    elif autogroup_mode == AUTOGROUP_EXPLICIT:
        if groups < 1:
            raise ValueError('Requested grouped convolution with fewer than 1 groups')
        if group_layout == GROUP_NONE and groups != 1:
            raise ValueError('GroupLayout not specified for grouped convolution')
        if groups == 1:
            autogroup_mode = AUTOGROUP_UNGROUPED
    elif autogroup_mode == AUTOGROUP_DEPTHWISE:
        if group_layout == GROUP_NONE:
            raise ValueError('Convolution GroupLayout must be specified to use DEPTHWISE AutoGroupMode')
    else:
        raise ValueError('Unrecognized AutoGroupMode')

    I = I_or_O if deriv_mode != DERIV_DATA else None
    F = F_or_O if deriv_mode != DERIV_FILTER else None
    O = I_or_O if deriv_mode == DERIV_DATA else (F_or_O if deriv_mode == DERIV_FILTER else None)

    def split_data(t):
        sh = list(t.shape)
        if len(sh) != rank + 2:
            raise ValueError('Inconsistent spatial rank in conv op (data tensor)')
        return (sh[0], sh[1], sh[2:]) if input_layout == LAYOUT_NCX else (sh[0], sh[-1], sh[1:-1])

    # what binding the tensors' dims yields
    N = CI = CO = G = F_CI = F_CO = None
    I_sp = O_sp = F_sp = None
    if I is not None:
        N, CI, I_sp = split_data(I)
    if O is not None:
        N, CO, O_sp = split_data(O)
    if F is not None:
        sh = list(F.shape)
        if len(sh) != rank + (3 if separate else 2):
            raise ValueError('Inconsistent spatial rank in conv op (filter tensor)')
        if filter_layout in (LAYOUT_GKCX, LAYOUT_KCX):
            if separate:
                G, sh = sh[0], sh[1:]
            F_CO, F_CI, F_sp = sh[0], sh[1], sh[2:]
        else:
            F_sp = sh[:rank]
            if separate:
                G = sh[rank]
            F_CI, F_CO = sh[-2], sh[-1]
        if filter_shape and list(filter_shape) != list(F_sp):
            raise ValueError('bind dims mismatch: filter_shape %s != %s' % (list(filter_shape), F_sp))
    if autogroup_mode in (AUTOGROUP_UNGROUPED, AUTOGROUP_EXPLICIT):
        if G is not None and G != groups:
            raise ValueError('bind dims mismatch: groups')
        G = groups
    elif autogroup_mode == AUTOGROUP_DEPTHWISE:
        # G is the dim CI itself; IN_K and SEPARATE also pin the filter's input channels to 1
        if group_layout in (GROUP_IN_K, GROUP_SEPARATE) and F_CI is not None and F_CI != 1:
            raise ValueError('bind dims mismatch: depthwise filter input channels')
        if group_layout == GROUP_IN_C and CI is None:
            CI = F_CI
        if CI is None:
            raise ValueError('unbound dimension CI')
        if G is not None and G != CI:
            raise ValueError('bind dims mismatch: groups')
        G = CI
    if G is None:
        raise ValueError('unbound dimension G')
    # channel dims shared with, or derived from, the filter's (ops.cc:1063-1083, 1184-1199)
    def same(a, b, what):
        if a is not None and b is not None and a != b:
            raise ValueError('bind dims mismatch: %s %d != %d' % (what, a, b))
        return a if a is not None else b
    if group_layout == GROUP_NONE:
        CO, CI = same(CO, F_CO, 'CO'), same(CI, F_CI, 'CI')
        F_CO, F_CI = CO, CI
    elif group_layout == GROUP_IN_C:
        CI = same(CI, F_CI, 'CI')
        F_CI = CI
        if F_CO is not None:
            CO = F_CO * G
    elif group_layout == GROUP_IN_K:
        CO = same(CO, F_CO, 'CO')
        F_CO = CO
        if F_CI is not None:
            CI = F_CI * G
    else:
        if F_CO is not None:
            CO = F_CO * G
        if F_CI is not None:
            CI = F_CI * G
    if deriv_mode == DERIV_FILTER:
        # the filter's channel extents are whatever stayed unbound-but-derivable in the reference: only the
        # layouts whose filter dims alias the data dims can be computed
        if group_layout == GROUP_NONE:
            F_CO, F_CI = CO, CI
        elif group_layout == GROUP_IN_C:
            F_CI = CI
        elif group_layout == GROUP_IN_K:
            F_CO = CO
        if F_CO is None or F_CI is None:
            raise ValueError('unbound filter channel dimension')
    if CI is None or CO is None:
        raise ValueError('unbound channel dimension')

    pads = []
    if deriv_mode == DERIV_NONE:
        O_sp = []
    if deriv_mode == DERIV_DATA:
        I_sp = []
    for i in range(rank):
        if deriv_mode == DERIV_DATA and not result_shape:
            p, size = compute_padding_and_input_size(O_sp[i], F_sp[i], strides[i], autopad, manual_padding[i],
                                                     manual_padding[i + rank], dilations[i], data_dilations[i])
            pads.append(p)
            I_sp.append(size)
            continue
        if deriv_mode == DERIV_FILTER and not result_shape:
            raise ValueError('Result shape inference not yet supported for filter transposed/derivative convolutions')
        in_size = result_shape[i] if deriv_mode == DERIV_DATA else I_sp[i]
        f_size = result_shape[i] if deriv_mode == DERIV_FILTER else F_sp[i]
        p, o = compute_padding_and_output_size(in_size, f_size, strides[i], autopad, manual_padding[i],
                                               manual_padding[i + rank], dilations[i], data_dilations[i])
        pads.append(p)
        if deriv_mode == DERIV_NONE:
            O_sp.append(o)
        if deriv_mode == DERIV_DATA:
            I_sp.append(result_shape[i])

    n, co, ci, g = E.TensorIndexes(4)
    x = E.TensorIndexes(rank)
    k = E.TensorIndexes(rank)
    grouped = group_layout != GROUP_NONE
    sp = [(strides[i] * x[i] + dilations[i] * k[i] - pads[i]) // data_dilations[i] for i in range(rank)]
    i_idxs = _data_order(input_layout, n, (CI // G) * g + ci if grouped else ci, sp)
    o_idxs = _data_order(input_layout, n, (CO // G) * g + co if grouped else co, x)
    f_co, f_ci, cons = co, ci, []
    if group_layout == GROUP_IN_C:
        f_ci = (CI // G) * g + ci
        cons.append(ci < CI // G)
    elif group_layout == GROUP_IN_K:
        f_co = (CO // G) * g + co
        cons.append(co < CO // G)
    f_idxs = _filter_order(filter_layout, g, f_co, f_ci, k)
    if deriv_mode == DERIV_NONE:
        c = E.Contraction(name).outShape(_data_order(input_layout, N, CO, O_sp)).outAccess(o_idxs)
        c.sum(I[i_idxs] * F[f_idxs])
    elif deriv_mode == DERIV_DATA:
        c = E.Contraction(name).outShape(_data_order(input_layout, N, CI, I_sp)).outAccess(i_idxs)
        c.sum(O[o_idxs] * F[f_idxs])
    else:
        c = E.Contraction(name).outShape(_filter_order(filter_layout, G, F_CO, F_CI, result_shape)).outAccess(f_idxs)
        c.sum(I[i_idxs] * O[o_idxs])
    return c.add_constraints(cons).build()


def pool(I, mode, pool_size, strides, autopad=VALID, manual_padding=None, include_padding_in_avg=False,
         use_ceil=False, name='pool'):
    rank = len(pool_size)
    manual_padding = list(manual_padding or [])
    while len(manual_padding) < 2 * rank:
        manual_padding.append(0)
    N, C = I.shape[0], I.shape[-1]
    X = I.shape[1:-1]
    n, c = E.TensorIndexes(2)
    x = E.TensorIndexes(rank)
    k = E.TensorIndexes(rank)
    o_dims, i_idxs, cons = [N], [n], []
    for i in range(rank):
        p, o = compute_padding_and_output_size(X[i], pool_size[i], strides[i], autopad, manual_padding[i],
                                               manual_padding[rank + i], 1, 1, use_ceil)
        o_dims.append(o)
        i_idxs.append(strides[i] * x[i] + k[i] - p)
        cons.append(k[i] < pool_size[i])
    o_dims.append(C)
    i_idxs.append(c)
    o_idxs = [n] + x + [c]

    def mk():
        return E.Contraction(name).outShape(o_dims).outAccess(o_idxs).add_constraints(cons)

    if mode == 'max':
        return mk().max(I[i_idxs]).build()
    if mode == 'min':
        return mk().min(I[i_idxs]).build()
    if mode == 'sum':
        return mk().sum(I[i_idxs]).build()
    if mode == 'avg':
        O = mk().sum(I[i_idxs]).build()
        if include_padding_in_avg:
            total = 1
            for s in pool_size:
                total *= s
            return O / total
        one = E.cast(E.Constant(1), I.dt)
        ones = E.Contraction(name).outShape(I.shape).outAccess(o_idxs).assign(one[()]).build()
        count = mk().sum(ones[i_idxs]).build()
        return O / count
    raise ValueError('Unrecognized pool_mode in pool op')


def dot(X, Y, name='dot'):
    if X.dt != Y.dt:
        raise ValueError('Invalid dtype in dot')
    if len(X.shape) == 1 and len(Y.shape) == 1:
        i, = E.TensorIndexes(1)
        return E.Contraction(name).outShape(X.shape[0]).outAccess(i).sum(X[i] * Y[i]).build()
    xi = E.TensorIndexes(len(X.shape))
    yi = E.TensorIndexes(len(Y.shape))
    z, = E.TensorIndexes(1)
    xi[-1] = z
    yi[-2] = z
    o_dims = list(X.shape[:-1]) + list(Y.shape[:-2]) + [Y.shape[-1]]
    o_idxs = xi[:-1] + yi[:-2] + [yi[-1]]
    return E.Contraction(name).outShape(o_dims).outAccess(o_idxs).sum(X[xi] * Y[yi]).build()


class _Axes:
    """AggregationAxes, plaidml/op/lib/ops.cc:71-127."""

    def __init__(self, shape, axes, keepdims):
        nd = len(shape)
        if axes is None:
            axes = list(range(nd))
        if isinstance(axes, int):
            axes = [axes]
        self.axes = sorted(set(a + nd if a < 0 else a for a in axes))
        self.src_idxs = E.TensorIndexes(nd)
        self.src_dims = list(shape)
        self.reduce_idxs = [self.src_idxs[a] for a in self.axes]
        self.reduce_dims = [shape[a] for a in self.axes]
        if keepdims:
            self.dst_idxs = list(self.src_idxs)
            self.dst_dims = list(shape)
            for a in self.axes:
                self.dst_idxs[a] = E.TensorIndex()
                self.dst_dims[a] = 1
        else:
            self.dst_idxs = [self.src_idxs[i] for i in range(nd) if i not in self.axes]
            self.dst_dims = [shape[i] for i in range(nd) if i not in self.axes]


def _reduce(I, axes, keepdims, agg, name):
    a = _Axes(I.shape, axes, keepdims)
    c = E.Contraction(name).outShape(a.dst_dims).outAccess(a.dst_idxs)
    getattr(c, agg)(I[a.src_idxs])
    return c.build(), a


def sum(I, axes=None, keepdims=False):  # noqa: A001
    return _reduce(I, axes, keepdims, 'sum', 'sum')[0]


def max(I, axes=None, keepdims=False):  # noqa: A001
    return _reduce(I, axes, keepdims, 'max', 'max')[0]


def min(I, axes=None, keepdims=False):  # noqa: A001
    return _reduce(I, axes, keepdims, 'min', 'min')[0]


def clip(I, lo, hi):
    """plaidml/op/lib/ops.cc:584-606: select(O > lo, O, cast(lo)) then select(O < hi, O, cast(hi))."""
    O = I
    if lo is not None:
        O = E.select(O > lo, O, E.cast(lo, O.dt))
    if hi is not None:
        O = E.select(O < hi, O, E.cast(hi, O.dt))
    return O


def maximum(X, Y):
    return E.select(X < Y, Y, X)  # plaidml/op/lib/ops.cc:1958-1968


def minimum(X, Y):
    return E.select(X < Y, X, Y)


def mean(I, axes=None, keepdims=False):
    if len(I.shape) == 0 or (isinstance(axes, (list, tuple)) and len(axes) == 0):
        return I
    so, a = _reduce(I, axes, keepdims, 'sum', 'mean')
    denom = 1
    for ax in a.axes:
        denom *= I.shape[ax]
    return so / denom


def relu(I):
    return E.relu(I)


def softmax(I, axis=-1, name='softmax'):
    nd = len(I.shape)
    if axis < 0:
        axis += nd
    if axis != nd - 1:
        raise NotImplementedError('softmax over a non-trailing axis')
    idxs = E.TensorIndexes(nd)
    r_dims = list(I.shape)
    r_idxs = list(idxs)
    r_dims[axis] = 1
    r_idxs[axis] = 0
    M = E.Contraction(name).outShape(r_dims).outAccess(r_idxs).max(I[idxs]).build()
    Ex = E.exp(I - M)
    Nn = E.Contraction(name).outShape(r_dims).outAccess(r_idxs).sum(Ex[idxs]).build()
    return Ex / Nn


def argmax(I, axis=-1):
    a = _Axes(I.shape, axis, False)
    M = E.Contraction('argmax').outShape(a.dst_dims).outAccess(a.dst_idxs).max(I[a.src_idxs]).build()
    IX = E.index(a.reduce_dims, 0)
    AM = E.Contraction('argmax').outShape(a.dst_dims).outAccess(a.dst_idxs).max(
        E.cond(I[a.src_idxs], M[a.dst_idxs], IX[a.reduce_idxs])).build()
    return E.cast(AM, E.DType.UINT32)


# ---------------------------------------------------------------------------
# Data movement and simple arithmetic of the operation library, each restated as the single
# contraction / elementwise chain the reference builds (plaidml/op/lib/ops.cc, lines per function).
# ---------------------------------------------------------------------------
PAD_CONSTANT, PAD_EDGE, PAD_REFLECT, PAD_SYMMETRIC = range(4)
LAYOUT_NXC, LAYOUT_NCX = 0, 1
AUTO_DIM_MATCH, AUTO_DIM_FILL = 0, -1


def _axis(axis, nd, what):
    if axis < -nd or axis >= nd:
        raise ValueError('axis out of range in %s: %d for a tensor of rank %d' % (what, axis, nd))
    return axis + nd if axis < 0 else axis


def _axis_list(axes):
    return [axes] if isinstance(axes, int) else list(axes)


def abs(I):  # noqa: A001
    return E.select(I < 0.0, -I, I)  # ops.cc:439-447


def concatenate(tensors, axis):
    """ops.cc:608-668: every input assigned at its offset into an otherwise zero result; the results added."""
    tensors = list(tensors)
    nd = len(tensors[0].shape)
    axis = _axis(axis, nd, 'concatenate')
    dims = list(tensors[0].shape)
    dims[axis] = builtins.sum(t.shape[axis] for t in tensors)
    idxs = E.TensorIndexes(nd)
    out, off = None, 0
    for t in tensors:
        o_idxs = list(idxs)
        o_idxs[axis] = idxs[axis] + off
        r = E.Contraction('concatenate').outShape(dims).outAccess(o_idxs).assign(t[idxs]).build()
        out = r if out is None else out + r
        off += t.shape[axis]
    return out


def cumsum(I, axis, exclusive=False):
    """ops.cc:1490-1510: O[.., i, ..] += I[.., i - k (- 1), ..] for 0 <= k < dim."""
    nd = len(I.shape)
    axis = _axis(axis, nd, 'cumsum')
    o_idxs = E.TensorIndexes(nd)
    i_idxs = list(o_idxs)
    k = E.TensorIndex()
    i_idxs[axis] = o_idxs[axis] - k - 1 if exclusive else o_idxs[axis] - k
    return E.Contraction('cumsum').outShape(I.shape).outAccess(o_idxs).sum(I[i_idxs]).add_constraint(k < I.shape[axis]).build()


def elu(I, alpha):
    return E.select(I < 0.0, alpha * E.exp(I) - alpha, I)  # ops.cc:1563-1584


def explicit_padding(I, lo_pads, hi_pads, mode=PAD_CONSTANT, padval=0):
    """ops.cc:1586-1685: CONSTANT = assign at the offset into a result initialised with padval; EDGE = per
    dimension, the first / last slice repeated and joined around the tensor."""
    nd = len(I.shape)
    if len(lo_pads) != nd or len(hi_pads) != nd:
        raise ValueError('Inconsistent shapes in explicit_padding op')
    idxs = E.TensorIndexes(nd)
    if mode == PAD_CONSTANT:
        o_dims = [I.shape[i] + lo_pads[i] + hi_pads[i] for i in range(nd)]
        o_idxs = [idxs[i] + lo_pads[i] for i in range(nd)]
        pv = padval if isinstance(padval, E.Tensor) else E.Constant(padval)
        return E.Contraction('explicit_padding').outShape(o_dims).outAccess(o_idxs).assign(I[idxs]).init(pv).build()
    if mode == PAD_EDGE:
        O = I
        for i in range(nd):
            dst = E.TensorIndexes(nd)
            src_lo, src_hi = list(dst), list(dst)
            src_lo[i] = 0
            src_hi[i] = O.shape[i] - 1
            lo_dims, hi_dims = list(O.shape), list(O.shape)
            lo_dims[i], hi_dims[i] = lo_pads[i], hi_pads[i]
            Lo = E.Contraction('explicit_padding').outShape(lo_dims).outAccess(dst).assign(O[src_lo]).build()
            Hi = E.Contraction('explicit_padding').outShape(hi_dims).outAccess(dst).assign(O[src_hi]).build()
            O = concatenate([Lo, O, Hi], i)
        return O
    raise NotImplementedError('padding mode %d' % mode)


def flip(I, axis=None):
    """ops.cc:1687-1725: O[.., dim - 1 - i, ..] = I[.., i, ..]."""
    nd = len(I.shape)
    axes = range(nd) if axis is None else [_axis(a, nd, 'flip') for a in _axis_list(axis)]
    i_idxs = E.TensorIndexes(nd)
    o_idxs = list(i_idxs)
    for a in axes:
        o_idxs[a] = I.shape[a] - 1 - i_idxs[a]
    return E.Contraction('flip').outShape(I.shape).outAccess(o_idxs).assign(I[i_idxs]).build()


def hard_sigmoid(I, slope):
    """ops.cc:1803-1820."""
    if slope <= 0:
        raise ValueError('hard_sigmoid expects positive slope')
    hi_cusp = 1.0 / (2.0 * slope)
    lo = E.cast(E.Constant(0.0), I.dt)
    hi = E.cast(E.Constant(1.0), I.dt)
    return E.select(I < -hi_cusp, lo, E.select(I > hi_cusp, hi, slope * I + 0.5))


def prod(I, axes=None, keepdims=False):
    return _reduce(I, axes, keepdims, 'product', 'prod')[0]  # ops.cc:2532-


def repeat(I, repeats, axis):
    """ops.cc:2782-2819: O[.., r * i + k, ..] = I[.., i, ..] for 0 <= k < r."""
    nd = len(I.shape)
    axis = _axis(axis, nd, 'repeat')
    o_dims = list(I.shape)
    o_dims[axis] = repeats * I.shape[axis]
    i_idxs = E.TensorIndexes(nd)
    o_idxs = list(i_idxs)
    k = E.TensorIndex()
    o_idxs[axis] = repeats * i_idxs[axis] + k
    return E.Contraction('repeat').outShape(o_dims).outAccess(o_idxs).assign(I[i_idxs]).add_constraint(k < repeats).build()


def reshape(I, dims):
    """ops.cc:2821-2885: 0 / None take the input's dimension, -1 is inferred from the element count."""
    out, fill = [], None
    for i, d in enumerate(dims):
        if d is None or d == AUTO_DIM_MATCH:
            if i >= len(I.shape):
                raise ValueError('matching dimension requested at %d from %d-dimensional tensor' % (i + 1, len(I.shape)))
            out.append(I.shape[i])
        elif d == AUTO_DIM_FILL:
            if fill is not None:
                raise ValueError("at most one dimension's size may be inferred")
            fill = i
            out.append(1)
        else:
            out.append(int(d))
    if fill is not None:
        num = den = 1
        for d in I.shape:
            num *= d
        for d in out:
            den *= d
        out[fill] = num // den
    return E.reshape(I, out)


def sigmoid(I):
    return 1.0 / (1.0 + E.exp(-I))  # ops.cc:2906-2915


def spatial_padding(I, lo_pads, hi_pads, layout=LAYOUT_NXC):
    """ops.cc:3129-: zero padding of the spatial dimensions (NXC / NCX)."""
    nd = len(I.shape)
    first = 1 if layout == LAYOUT_NXC else 2
    if len(lo_pads) != nd - 2 or len(hi_pads) != nd - 2:
        raise ValueError('Inconsistent spatial rank in spatial_padding op')
    i_idxs = E.TensorIndexes(nd)
    o_dims, o_idxs = list(I.shape), list(i_idxs)
    for i in range(nd - 2):
        o_dims[first + i] = I.shape[first + i] + lo_pads[i] + hi_pads[i]
        o_idxs[first + i] = i_idxs[first + i] + lo_pads[i]
    return E.Contraction('spatial_padding').outShape(o_dims).outAccess(o_idxs).assign(I[i_idxs]).build()


def square(I):
    return I * I  # ops.cc:3380-3384


def squeeze(I, axes):
    nd = len(I.shape)
    drop = {_axis(a, nd, 'squeeze') for a in _axis_list(axes)}
    return E.reshape(I, [I.shape[i] for i in range(nd) if i not in drop])  # ops.cc:3386-3422


def tile(I, tiling_factors):
    """ops.cc:3454-3489: O[.., t * dim + i, ..] = I[.., i, ..] for every repetition t."""
    nd = len(I.shape)
    reps = list(tiling_factors) + [1] * (nd - len(tiling_factors))
    if not tiling_factors or len(reps) > nd:
        raise ValueError('bad tiling factors')
    i_idxs = E.TensorIndexes(nd)
    o_dims = [I.shape[i] * reps[i] for i in range(nd)]
    o_idxs = [E.TensorIndex() * I.shape[i] + i_idxs[i] for i in range(nd)]
    return E.Contraction('tile').outShape(o_dims).outAccess(o_idxs).assign(I[i_idxs]).build()


def transpose(I, axes=None):
    """ops.cc:3491-3537: dimension i of the output is dimension axes[i] of the input (default: reversed)."""
    nd = len(I.shape)
    pattern = list(range(nd - 1, -1, -1)) if axes is None else list(axes)
    i_idxs = E.TensorIndexes(nd)
    return E.Contraction('transpose').outShape([I.shape[p] for p in pattern]).outAccess([i_idxs[p] for p in pattern]) \
        .assign(I[i_idxs]).build()


def unsqueeze(I, axes):
    axes = _axis_list(axes)
    nd = len(I.shape) + len(axes)
    new = {_axis(a, nd, 'unsqueeze') for a in axes}
    src = iter(I.shape)
    return E.reshape(I, [1 if i in new else next(src) for i in range(nd)])  # ops.cc:3539-3584 (same element order)


def variance(I, axes=None, keepdims=False):
    """ops.cc:3586-3632: mean of squared differences from the mean (denominator n)."""
    M = mean(I, axes, True)
    d2 = (I - M) * (I - M)
    so, a = _reduce(d2, axes, keepdims, 'sum', 'variance')
    denom = 1
    for ax in a.axes:
        denom *= I.shape[ax]
    return so / denom


EPS_ADD, EPS_MAX = range(2)


def _truth(I):
    one = E.cast(1, I.dt)
    zero = E.cast(0, I.dt)
    return E.select(I == 0, zero, one), zero, one


def all(I, axes=None, keepdims=False):  # noqa: A001
    """ops.cc:450-475: product of the 0 / 1 image of the input, as UINT8."""
    T, zero, one = _truth(I)
    if len(I.shape) == 0 or (isinstance(axes, (list, tuple)) and len(axes) == 0):
        return E.cast(T, E.DType.UINT8)
    return E.cast(_reduce(T, axes, keepdims, 'product', 'all')[0], E.DType.UINT8)


def any(I, axes=None, keepdims=False):  # noqa: A001
    """ops.cc:477-503: sum of the 0 / 1 image, compared with 0, as UINT8."""
    T, zero, one = _truth(I)
    if len(I.shape) == 0 or (isinstance(axes, (list, tuple)) and len(axes) == 0):
        return E.cast(T, E.DType.UINT8)
    S = _reduce(T, axes, keepdims, 'sum', 'any')[0]
    return E.cast(E.select(S == 0, zero, one), E.DType.UINT8)


def binary_crossentropy(targets, preds, epsilon):
    """ops.cc:523-544."""
    if epsilon < 0. or epsilon >= 0.5:
        raise ValueError('The epsilon used in binary_crossentropy must be between 0 and 0.5, received %s' % epsilon)
    P = clip(preds, float(epsilon), 1. - float(epsilon))
    return -targets * E.log(P) - (1 - targets) * E.log(1 - P)


def broadcast(I, result_shape, bcast_axes):
    """ops.cc:546-582."""
    if len(I.shape) != len(bcast_axes):
        raise ValueError('Mismatched broadcast axes')
    o_idxs = E.TensorIndexes(len(result_shape))
    i_idxs = [0 if I.shape[i] == 1 else o_idxs[a] for i, a in enumerate(bcast_axes)]
    return E.Contraction('broadcast').outShape(list(result_shape)).outAccess(o_idxs).assign(I[i_idxs]).build()


def cumprod(I, axis):
    """ops.cc:1469-1488."""
    nd = len(I.shape)
    axis = _axis(axis, nd, 'cumprod')
    o_idxs = E.TensorIndexes(nd)
    i_idxs = list(o_idxs)
    k = E.TensorIndex()
    i_idxs[axis] = o_idxs[axis] - k
    return E.Contraction('cumprod').outShape(I.shape).outAccess(o_idxs).product(I[i_idxs]).add_constraint(k < I.shape[axis]).build()


def l2norm(I, axes, epsilon=0.0, eps_mode=EPS_ADD):
    """ops.cc:2505-2530."""
    X = sum(I * I, list(axes), True)
    if eps_mode == EPS_ADD:
        X = X + float(epsilon)
    elif eps_mode == EPS_MAX:
        X = maximum(X, E.cast(float(epsilon), X.dt))
    else:
        raise ValueError('Unrecognized eps_mode in l2norm op')
    return E.sqrt(X)


def lrn(I, window_size, axes=(-1,), alpha=1.0, beta=1.0, epsilon=1e-5):
    """ops.cc:129-160, 1920-1941: the window over axis a covers offsets -w/2 .. w - 1 - w/2 (integer division)."""
    nd = len(I.shape)
    ax = sorted(set(a + nd if a < 0 else a for a in axes))
    if len(ax) != len(window_size):
        raise ValueError('Inconsistent axis count and window width count in LRN')
    dst = E.TensorIndexes(nd)
    src = list(dst)
    c = E.Contraction('lrn').outShape(I.shape).outAccess(dst)
    cons = []
    for a, w in zip(ax, window_size):
        k = E.TensorIndex()
        cons.append(k < int(w))
        src[a] = dst[a] + k - int(w) // 2
    c.sum((I * I)[src])
    for k in cons:
        c.add_constraint(k)
    return I / E.pow(float(alpha) * c.build() + float(epsilon), float(beta))


def mvn(I, axes=None, normalize_variance=True, epsilon=1e-9, across_channels=True, layout=''):
    """ops.cc:2469-2503."""
    if axes is None:
        if not layout:
            raise ValueError('Either axes or layout must be specified for MVN')
        axes = [i for i, d in enumerate(layout) if d != 'N' and not (d == 'C' and not across_channels)]
    R = I - mean(I, axes, True)
    if normalize_variance:
        stdev = E.sqrt(variance(I, axes, True))
        R = R / maximum(stdev, E.cast(float(epsilon), I.dt))
    return R


def reorg_yolo(I, stride, decrease, layout='NCHW'):
    """ops.cc:2730-2780, written for NCHW and permuted for any other arrangement of those four letters."""
    if len(I.shape) != 4:
        raise ValueError('PlaidML reorg_yolo op expects I to have 4 dimensions')
    perm = [layout.index(ch) for ch in 'NCHW']       # position of N, C, H, W in the tensor's layout
    N, C, H, W = (I.shape[p] for p in perm)
    s = int(stride)

    def place(vals):                                    # NCHW-ordered values -> the tensor's own order
        out = [None] * 4
        for v, p in zip(vals, perm):
            out[p] = v
        return out

    b, i, j, k, x, y = E.TensorIndexes(6)
    h = j * s + y
    w = i * s + x
    if decrease:
        c_out = C // (s * s)
        c = k + ((x + y * s) * c_out)
        con = E.Contraction('reorg_yolo').outShape(place([N, c_out, H * s, W * s])).outAccess(place([b, k, h, w]))
        con.assign(I[place([b, c, j, i])])
    else:
        c = k + ((x + y * s) * C)
        con = E.Contraction('reorg_yolo').outShape(place([N, C * s * s, H // s, W // s])).outAccess(place([b, c, j, i]))
        con.assign(I[place([b, k, h, w])])
    return con.add_constraint(y < s).add_constraint(x < s).build()


def scale_gradient(I, scale=-1.0):
    return I  # ops.cc:2888-2904: identity on the forward pass


def slice_of(I, slices):
    """ops.cc:2917-3047 (entries: int or Python slice, plaidml/op/__init__.py:246-257)."""
    nd = len(I.shape)
    if nd == 0:
        return I
    if len(slices) != nd:
        raise ValueError('%d slice axes provided to slice %d-dimensional tensor' % (len(slices), nd))
    o_idxs, o_dims, i_idxs = [], [], []
    for d, sl in enumerate(slices):
        dim = I.shape[d]
        if isinstance(sl, int):
            i_idxs.append(sl + dim if sl < 0 else sl)
            continue
        step = 1 if sl.step is None else int(sl.step)
        if step == 0:
            raise ValueError('Cannot slice with step size 0')
        if sl.start is None:
            start = 0 if step > 0 else dim - 1
        else:
            start = dim + sl.start if sl.start < 0 else sl.start
        if sl.stop is None:
            stop = dim if step > 0 else -1
        else:
            stop = dim + sl.stop if sl.stop < 0 else sl.stop
        to_ceil = step - 1 if step > 0 else step + 1
        num = stop - start + to_ceil
        o_dims.append(int(num / step) if num % step else num // step)  # C division: toward zero
        o = E.TensorIndex()
        o_idxs.append(o)
        i_idxs.append(start + step * o)
    return E.Contraction('slice').outShape(o_dims).outAccess(o_idxs).assign(I[i_idxs]).build()


TOPK_VALUE, TOPK_INDEX = range(2)


def gatherND(x, y, batch_dims=0, interpolation_mode=E.INTERP_NONE):
    """ops.cc:1728-1801: the ND mode of gather; LINEAR pads the addressed dimensions with two zeros per side and sums
    the 2^k corners of the surrounding cell weighted by the opposite distances."""
    idx_dims = y.shape[-1]
    if idx_dims + batch_dims > len(x.shape):
        raise ValueError('Invalid Indices')
    if interpolation_mode == E.INTERP_NONE:
        return E.gather(x, y, mode=E.GATHER_ND, batch_dims=batch_dims)
    if interpolation_mode != E.INTERP_LINEAR:
        raise ValueError('Unsupported InterpolationMode in gatherND')
    pads = [0] * len(x.shape)
    for i in range(idx_dims):
        pads[i + batch_dims] = 2
    X = explicit_padding(x, pads, pads, PAD_CONSTANT, 0)
    Y = y + 2
    if len(y.shape) - batch_dims != 2:
        raise ValueError('Indices dimension should be batch_dims plus two in interpolated gatherND')
    Yf = E.cast(Y, E.DType.FLOAT32)
    dims = [E.gather(Yf, E.cast(E.index([1], 0), E.DType.INT32) + i, axis=-1) for i in range(idx_dims)]
    lower = [E.floor(d) for d in dims]
    upper = [E.floor(d) + 1.0 for d in dims]
    zero = E.cast(E.index([1], 0), E.DType.FLOAT32)
    result = zero
    for corner in range(2 ** idx_dims):
        at, coeff, j = [], zero + 1, corner
        for k in range(idx_dims):
            high = j % 2
            j //= 2
            at.append(upper[k] if high else lower[k])
            coeff = coeff * squeeze(dims[k] - lower[k], [-1]) if high else coeff * squeeze(upper[k] - dims[k], [-1])
        vertex = E.gather(X, E.cast(concatenate(at, -1), E.DType.INT32), mode=E.GATHER_ND, batch_dims=batch_dims)
        result = result + vertex * broadcast(coeff, list(vertex.shape), list(range(len(coeff.shape))))
    return result


def _sorted_by(I, order, axis):
    nd = len(I.shape)
    coords = [unsqueeze(order if i == axis else E.index(list(order.shape), i), [nd]) for i in range(nd)]
    return E.gather(I, concatenate(coords, -1), mode=E.GATHER_ND)


def sort(I, axis=-1, direction=E.SORT_ASC):
    """ops.cc:3100-3127."""
    axis = _axis(axis, len(I.shape), 'sort')
    return _sorted_by(I, E.argsort(I, axis, direction), axis)


def topk(I, k, axis=-1, sort_direction=E.SORT_DESC, sort_type=TOPK_VALUE, index_element_type=None):
    """ops.cc:2420-2467; returns (values, positions)."""
    axis = _axis(axis, len(I.shape), 'topk')
    order = E.argsort(I, axis, sort_direction)
    first_k = E.index([int(k)], 0)
    idxs = E.gather(order, first_k, axis=axis)
    if sort_type == TOPK_VALUE:
        return E.gather(_sorted_by(I, order, axis), first_k, axis=axis), idxs
    by_position = _sorted_by(idxs, E.argsort(idxs, axis, E.SORT_ASC), axis)
    return _sorted_by(I, by_position, axis), by_position


RESIZE_NEAREST, RESIZE_BILINEAR = range(2)


def image_resize(I, factors, interp=RESIZE_NEAREST, layout=LAYOUT_NXC):
    """ops.cc:1822-1918: NEAREST repeats pixels; BILINEAR spreads every pixel with a (2f-1) x (2f-1) tent kernel
    (corners aligned to 0 and f * (dim - 1), zero outside)."""
    if builtins.any(f <= 0 for f in factors):
        raise ValueError('All scaling factors in image_resize must be positive')
    if len(I.shape) != 4 or len(factors) != 2:
        raise ValueError('image_resize expects 2 spatial dims and 2 factors')
    if layout not in (LAYOUT_NXC, LAYOUT_NCX):
        raise ValueError('Unable to apply image_resize to a tensor with this layout')
    pre = 2 if layout == LAYOUT_NCX else 1
    fh, fw = int(factors[0]), int(factors[1])
    if interp == RESIZE_NEAREST:
        return repeat(repeat(I, fh, pre), fw, pre + 1)
    if interp != RESIZE_BILINEAR:
        raise ValueError('Unrecognized InterpolationMode in image_resize')
    j, i, y, x = E.TensorIndexes(4)
    hcoef = E.cast(1.0 / fh, E.DType.FLOAT32)
    wcoef = E.cast(1.0 / fw, E.DType.FLOAT32)
    hvec = E.Contraction('image_resize').outShape([fh]).outAccess([y]).assign(hcoef[[]]).build()
    wvec = E.Contraction('image_resize').outShape([fw]).outAccess([x]).assign(wcoef[[]]).build()
    hk = E.Contraction('image_resize').outShape([2 * fh - 1]).outAccess([y]).sum(hvec[j + y - fh + 1]).add_constraint(j < fh).build()
    wk = E.Contraction('image_resize').outShape([2 * fw - 1]).outAccess([x]).sum(wvec[i + x - fw + 1]).add_constraint(i < fw).build()
    K = E.Contraction('image_resize').outShape([2 * fh - 1, 2 * fw - 1]).outAccess([y, x]).assign(hk[y] * wk[x]).build()
    idxs = E.TensorIndexes(4)
    o_dims, o_idxs = list(I.shape), list(idxs)
    o_dims[pre], o_dims[pre + 1] = fh * I.shape[pre], fw * I.shape[pre + 1]
    o_idxs[pre] = fh * idxs[pre] + j - fh + 1
    o_idxs[pre + 1] = fw * idxs[pre + 1] + i - fw + 1
    return E.Contraction('image_resize').outShape(o_dims).outAccess(o_idxs).sum(I[idxs] * K[j, i]).build()


BOXES_NMS, BOXES_SSD = range(2)
NMS_CAFFE, NMS_MXNET, NMS_OV = range(3)


def _box_corners(boxes, variances, location, decode, in_h, in_w, clip_boxes, centered):
    """decode_boxes, ops.cc:2034-2117: (y1, x1, y2, x2), each the box tensor without its last axis."""
    col = lambda t, k: E.gather(t, k, axis=3)  # noqa: E731
    if centered:
        if decode == BOXES_NMS:  # [x, y, width, height]
            xc, yc, hw, hh = col(boxes, 0), col(boxes, 1), col(boxes, 2) / 2.0, col(boxes, 3) / 2.0
        elif decode == BOXES_SSD:
            px1, py1 = col(boxes, 0) / in_w, col(boxes, 1) / in_h
            px2, py2 = col(boxes, 2) / in_w, col(boxes, 3) / in_h
            v = [col(variances, k) for k in range(4)]
            loc = [col(location, k) for k in range(4)]
            pw, ph = px2 - px1, py2 - py1
            xc = v[0] * loc[0] * pw + (px1 + px2) / 2.0
            yc = v[1] * loc[1] * ph + (py1 + py2) / 2.0
            hw = E.exp(v[2] * loc[2]) * pw / 2.0
            hh = E.exp(v[3] * loc[3]) * ph / 2.0
        else:
            raise ValueError('Unrecognized boxes decode mode')
        x1, x2, y1, y2 = xc - hw, xc + hw, yc - hh, yc + hh
    elif decode == BOXES_NMS:  # [y1, x1, y2, x2] with either corner first
        ya, xa, yb, xb = (col(boxes, k) for k in range(4))
        y1, x1, y2, x2 = minimum(ya, yb), minimum(xa, xb), maximum(ya, yb), maximum(xa, xb)
    elif decode == BOXES_SSD:  # [x1, y1, x2, y2]
        boxes = boxes / in_w + variances * location
        x1, y1, x2, y2 = (col(boxes, k) for k in range(4))
    else:
        raise ValueError('Unrecognized boxes decode mode')
    if clip_boxes:
        lo, hi = E.cast(0.0, E.DType.FLOAT32), E.cast(1.0, E.DType.FLOAT32)
        y1, x1, y2, x2 = (clip(t, lo, hi) for t in (y1, x1, y2, x2))
    return [y1, x1, y2, x2]



def _pairwise_iou(corners, nb, nbox, nloc):
    """compute_iou, ops.cc:2119-2153: [batch, location class, box, box]."""
    zero = E.cast(E.index([1], 0), corners[0].dt)
    y1, x1, y2, x2 = (E.reshape(t, [nb, nloc, nbox]) for t in corners)
    area = (y2 - y1) * (x2 - x1)
    as_rows = lambda t: E.reshape(t, [nb, nloc, nbox, 1])  # noqa: E731
    as_cols = lambda t: E.reshape(t, [nb, nloc, 1, nbox])  # noqa: E731
    ygap = minimum(as_rows(y2), as_cols(y2)) - maximum(as_rows(y1), as_cols(y1))
    xgap = minimum(as_rows(x2), as_cols(x2)) - maximum(as_rows(x1), as_cols(x1))
    inter = E.select(ygap > 0.0, ygap, zero) * E.select(xgap > 0.0, xgap, zero)
    union = unsqueeze(area, [-1]) + unsqueeze(area, [-2]) - inter
    return inter * E.select(union <= 0.0, zero, 1.0 / union)


def nms(Boxes, Scores, iou_threshold, score_threshold, max_output_boxes_per_class, soft_nms_sigma=0.0,
        center_point_box=False, sort_result_descending=False, box_output_type=E.DType.INT32,
        boxes_decode_mode=BOXES_NMS, clip_before_nms=False, clip_after_nms=False, ssd_input_height=0,
        ssd_input_width=0, ssd_variances=None, ssd_location=None, ssd_with_arm_loc=False, ssd_arm_location=None,
        nms_style=NMS_OV, share_location=True, hard_suppression=True):
    """ops.cc:2157-2417.  Greedy non-maximum suppression unrolled max_output_boxes_per_class times over
    Scores [batch, class, box]: each round takes every (batch, class)'s best remaining box, records it, and zeroes
    the scores of the boxes that overlap it.  Returns [selected (batch, class, box) triples, (batch, class, score)
    triples, the number of valid selections]; unused rows are -1."""
    if boxes_decode_mode not in (BOXES_NMS, BOXES_SSD):
        raise ValueError('Invalid enumeration value')
    if nms_style not in (NMS_CAFFE, NMS_MXNET, NMS_OV):
        raise ValueError('Invalid enumeration value')
    in_dt, thr_dt, out_dt = Boxes.dt, iou_threshold.dt, E.DType(box_output_type)
    nb, nc, nbox = Scores.shape
    nloc = 1 if share_location else nc

    zero = E.cast(E.index([1], 0), in_dt)
    zero_int = E.cast(zero, E.DType.INT32)
    one = zero + 1
    neg1 = -one
    neg1_o = E.cast(neg1, out_dt)
    valid_outputs = zero

    Boxes = unsqueeze(Boxes, [1])
    if ssd_with_arm_loc:
        ssd_variances = unsqueeze(ssd_variances, [1])
        p = _box_corners(Boxes, ssd_variances, ssd_arm_location, boxes_decode_mode, ssd_input_height, ssd_input_width,
                         clip_before_nms, center_point_box)
        priors = concatenate([p[1], p[0], p[3], p[2]], -1)
        corners = _box_corners(priors, ssd_variances, ssd_location, boxes_decode_mode, ssd_input_height,
                               ssd_input_width, clip_before_nms, center_point_box)
    else:
        if boxes_decode_mode == BOXES_SSD:
            ssd_variances = unsqueeze(ssd_variances, [1])
        corners = _box_corners(Boxes, ssd_variances, ssd_location, boxes_decode_mode, ssd_input_height,
                               ssd_input_width, clip_before_nms, center_point_box)
    iou = _pairwise_iou(corners, nb, nbox, nloc)
    weight = -0.5 / soft_nms_sigma if soft_nms_sigma != 0 else 0.0

    invalid_node = E.cast(E.Constant(np.array([[[-1, -1]]], np.float32), name='invalid_node'), out_dt)
    per_class = builtins.min(nbox, max_output_boxes_per_class) if max_output_boxes_per_class != 0 else nbox
    index_bc = E.cast(concatenate([E.index([nb, nc, 1], 0), E.index([nb, nc, 1], 1)], 2), out_dt)
    score_thr = E.cast(score_threshold, in_dt)
    iou_thr = E.cast(iou_threshold, in_dt)
    new_scores = E.select(Scores > score_thr, Scores, zero)

    def zeros(shape):
        return E.Contraction('nms').outShape(shape).outAccess(E.TensorIndexes(3)).assign(zero[0]).build()

    if nms_style == NMS_CAFFE:  # only the top scores of each class take part
        vals, idxs = topk(new_scores, per_class, axis=2)
        new_scores = E.scatter(zeros([nb, nc, nbox]), idxs, vals, axis=2, mode=E.SCATTER_UPDATE_ELT)
    elif nms_style == NMS_MXNET:  # each box competes in its best class only, and only the top boxes do
        best_class = squeeze(E.gather(E.argsort(new_scores, 1, E.SORT_DESC), 0, axis=1), [1])
        best_score = squeeze(E.gather(sort(new_scores, 1, E.SORT_DESC), 0, axis=1), [1])
        top_scores, top_boxes = topk(best_score, per_class, axis=1, sort_type=TOPK_INDEX)
        top_classes = gatherND(best_class, unsqueeze(top_boxes, [-1]), batch_dims=1)
        batch_idx = unsqueeze(E.index(list(top_classes.shape), 0), [-1])
        where = concatenate([batch_idx, unsqueeze(top_classes, [-1]), unsqueeze(top_boxes, [-1])], -1)
        new_scores = E.scatter(zeros([nb, nc, nbox]), where, top_scores, mode=E.SCATTER_UPDATE_ND)

    zero_cell = zeros([nb, nc, 1])
    boxes, scores = [], []
    for _ in range(per_class):
        candidate = E.gather(E.argsort(new_scores, 2, E.SORT_DESC), 0, axis=2)
        score = E.reshape(max(new_scores, 2), [nb, nc, 1])
        node = E.select(score > 0.0, index_bc, invalid_node)
        valid_outputs = valid_outputs + sum(E.select(score != 0.0, one, zero))
        scores.append(E.cast(node, thr_dt))
        score = E.select(score > 0.0, score, neg1)
        scores.append(E.cast(score, thr_dt))
        # the winner itself goes to zero by position (equal scores may exist), its neighbours by overlap
        new_scores = E.reshape(E.scatter(new_scores, candidate, zero_cell, axis=2, mode=E.SCATTER_UPDATE_ELT),
                               [nb, nc, nbox])
        if share_location:
            class_idx = broadcast(zero_int, list(candidate.shape), [1])
        else:
            class_idx = E.index(list(candidate.shape), 1)
        overlap = gatherND(iou, concatenate([class_idx, candidate], 2), batch_dims=1)
        suppressed = (overlap >= iou_thr) if hard_suppression else (overlap > iou_thr)
        new_scores = E.select(suppressed, zero, new_scores)
        box_index = E.select(score > 0.0, E.cast(candidate, out_dt), neg1_o)
        boxes.append(node)
        boxes.append(E.reshape(box_index, [nb, nc, 1]))
        if soft_nms_sigma != 0:
            new_scores = new_scores * E.exp(overlap * overlap * weight)
            new_scores = E.select(new_scores > score_thr, new_scores, zero)

    valid_outputs = E.cast(valid_outputs, out_dt)
    rows = nb * nc * per_class
    scores_result = E.reshape(concatenate(scores, 2), [rows, 3])
    boxes_result = E.reshape(concatenate(boxes, 2), [rows, 3])
    if sort_result_descending:
        order = E.argsort(E.reshape(E.gather(scores_result, 2, axis=1), [rows]), 0, E.SORT_DESC)
        scores_result = E.gather(scores_result, order, axis=0)
        boxes_result = E.gather(boxes_result, order, axis=0)
    else:
        # a stable sort on "position, or past-the-end for a -1" moves the unused entries to the back
        n = rows * 3
        flat_scores, flat_boxes = E.reshape(scores_result, [n]), E.reshape(boxes_result, [n])
        key = E.select(flat_scores != E.cast(-1, thr_dt), E.index([n], 0), E.cast(n, E.DType.INT32))
        order = E.argsort(E.cast(key, E.DType.FLOAT32), 0)
        scores_result = E.reshape(E.gather(flat_scores, order, axis=0), [rows, 3])
        boxes_result = E.reshape(E.gather(flat_boxes, order, axis=0), [rows, 3])
        if boxes_decode_mode == BOXES_SSD:
            decoded = concatenate([corners[1], corners[0], corners[3], corners[2]], -1)
            if clip_after_nms:
                decoded = clip(decoded, E.cast(0.0, E.DType.FLOAT32), E.cast(1.0, E.DType.FLOAT32))
            if share_location:
                pick = E.gather(boxes_result, concatenate([zero_int, zero_int + 2], 0), axis=1)
                out_boxes = gatherND(squeeze(decoded, [0]), pick)
            else:
                out_boxes = gatherND(decoded, boxes_result)
            if nms_style == NMS_MXNET:
                classes = E.gather(boxes_result, 1, axis=1) - 1  # drops the background class
                one_int = zero_int + 1
                scores_result = E.scatter(scores_result, one_int, E.cast(classes, scores_result.dt), axis=1,
                                          mode=E.SCATTER_UPDATE_SLICE)
                boxes_result = E.scatter(boxes_result, one_int, classes, axis=1, mode=E.SCATTER_UPDATE_SLICE)
            scores_result = concatenate([scores_result, out_boxes], 1)
    return [boxes_result, scores_result, valid_outputs]

"""Op-library subset of the CPU oracle -- TEST INFRASTRUCTURE ONLY.

Restates, on top of oracle/tile_oracle.py, the contractions that the reference
op library emits for the operations on the hot path (plaidml/op/lib/ops.cc):

  convolution   :879-1467 (NXC input, XCK filter; strides, dilations, autopad,
                 explicit padding, group layouts NONE and IN_C with DEPTHWISE
                 autogrouping), padding rule :347-382
  pool          :2562-2703 (MAX / MIN / SUM / AVG, NXC)
  dot           :1512-1561
  mean          :1970-2003, sum / max via the same AggregationAxes :71-127
  relu          :2705-2728 (plain form only)
  softmax       :3049-3098 (last-axis form)
  argmax        :505-521

Nothing in the shipped package imports this module.
"""
import builtins

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


def convolution(I, F, strides=None, dilations=None, data_dilations=None, autopad=SAME_UPPER,
                manual_padding=None, depthwise=False, name='conv'):
    """NXC input, XCK filter.  depthwise=True is GroupLayout IN_C + AutoGroupMode DEPTHWISE."""
    rank = len(I.shape) - 2
    strides = list(strides or [1] * rank)
    dilations = list(dilations or [1] * rank)
    data_dilations = list(data_dilations or [1] * rank)
    manual_padding = list(manual_padding or [])
    if len(manual_padding) == rank:
        manual_padding = manual_padding + manual_padding  # symmetric shorthand
    while len(manual_padding) < 2 * rank:
        manual_padding.append(0)
    if manual_padding and builtins.any(manual_padding) and autopad != EXPLICIT:
        raise ValueError('Autopadding and manual padding both requested for single conv operation')
    N, CI = I.shape[0], I.shape[-1]
    xs = I.shape[1:-1]
    ks = F.shape[:rank]
    F_CI, F_CO = F.shape[rank], F.shape[rank + 1]
    if F_CI != CI:
        raise ValueError('bind dims mismatch: filter input channels %d != %d' % (F_CI, CI))
    G = CI if depthwise else 1
    CO = F_CO * G if depthwise else F_CO
    n, co, ci, g = E.TensorIndexes(4)
    x = E.TensorIndexes(rank)
    k = E.TensorIndexes(rank)
    pads, outs = [], []
    for i in range(rank):
        p, o = compute_padding_and_output_size(xs[i], ks[i], strides[i], autopad, manual_padding[i],
                                               manual_padding[i + rank], dilations[i], data_dilations[i])
        pads.append(p)
        outs.append(o)
    sp = [(strides[i] * x[i] + dilations[i] * k[i] - pads[i]) // data_dilations[i] for i in range(rank)]
    cons = []
    if depthwise:
        i_c = (CI // G) * g + ci
        f_ci, f_co = (CI // G) * g + ci, co
        o_c = (CO // G) * g + co
        cons.append(ci < CI // G)
    else:
        i_c, f_ci, f_co, o_c = ci, ci, co, co
    c = E.Contraction(name).outShape([N] + outs + [CO]).outAccess([n] + x + [o_c])
    c.sum(I[[n] + sp + [i_c]] * F[k + [f_ci, f_co]]).add_constraints(cons)
    return c.build()


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

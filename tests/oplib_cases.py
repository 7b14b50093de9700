"""Cases for the data-movement / simple-arithmetic operations of the op library, each built twice (oracle
and product EDSL): name -> builder(E, op) returning (program, inputs, expected numpy result, exact?).

Expected values are numpy closed forms (np.concatenate, np.pad, np.cumsum, ...) and, where the reference holds
an exact case, that case (plaidml/op/op_test.cc: CumSumExclusive :297-304, ExplicitPadding :318-333,
ExplicitPaddingNegInf :335-351, ExplicitPaddingInf :353-370, ExplicitPaddingNoOp :372-383,
ExplicitPaddingEdge :385-418, Broadcast* :52-158, ReorgYoloDecrease / ReorgYoloIncrease :552-581 with their loop-nest
reference :524-550).  A case may return lists of outputs / expected arrays.
"""
import numpy as np


def _rng():
    return np.random.default_rng(77)


def _f32(E, shape):
    return E.Placeholder(E.DType.FLOAT32, list(shape))


def _one(E, name, shape, fn, data=None):
    X = _f32(E, shape)
    x = _rng().standard_normal(shape).astype(np.float32) if data is None else np.asarray(data, np.float32).reshape(shape)
    return E.Program(name, [X], [fn(X)]), [x], x


def concatenate(E, op):
    A, B, C = _f32(E, (2, 3, 4)), _f32(E, (2, 5, 4)), _f32(E, (2, 1, 4))
    r = _rng()
    a, b, c = (r.standard_normal(s).astype(np.float32) for s in ((2, 3, 4), (2, 5, 4), (2, 1, 4)))
    return E.Program('concatenate', [A, B, C], [op.concatenate([A, B, C], 1)]), [a, b, c], np.concatenate([a, b, c], 1), True


def cumsum(E, op):
    p, ins, x = _one(E, 'cumsum', (3, 5, 4), lambda X: op.cumsum(X, 1))
    return p, ins, np.cumsum(x.astype(np.float64), 1), False


def cumsum_exclusive_reference(E, op):
    p, ins, _ = _one(E, 'cumsum', (4,), lambda X: op.cumsum(X, 0, True), [2, 4, 6, 8])
    return p, ins, np.array([0, 2, 6, 12], np.float32), True


def _pad_ref(E, op, data, padval):
    X = _f32(E, (2, 3))
    O = op.explicit_padding(X, [2, 1], [2, 1], op.PAD_CONSTANT, E.Constant(padval))
    x = np.asarray(data, np.float32).reshape(2, 3)
    return E.Program('explicit_padding', [X], [O]), [x], np.pad(x, ((2, 2), (1, 1)), constant_values=padval), True


def explicit_padding_reference(E, op):
    return _pad_ref(E, op, [1, 2, 3, 4, 5, 6], -1.0)


def explicit_padding_neg_inf_reference(E, op):
    return _pad_ref(E, op, [1, 2, 3, 4, 5, 6], -np.inf)


def explicit_padding_inf_reference(E, op):
    return _pad_ref(E, op, [-1, -2, -3, -4, -5, -6], np.inf)


def explicit_padding_noop_reference(E, op):
    X = _f32(E, (2, 3))
    x = np.arange(1, 7, dtype=np.float32).reshape(2, 3)
    return E.Program('explicit_padding', [X], [op.explicit_padding(X, [0, 0], [0, 0], op.PAD_CONSTANT, E.Constant(0))]), [x], x, True


def explicit_padding_edge_reference(E, op):
    X = _f32(E, (1, 2, 3))
    x = np.arange(1, 7, dtype=np.float32).reshape(1, 2, 3)
    O = op.explicit_padding(X, [1, 2, 1], [2, 1, 3], op.PAD_EDGE)
    return E.Program('explicit_padding', [X], [O]), [x], np.pad(x, ((1, 2), (2, 1), (1, 3)), mode='edge'), True


def spatial_padding(E, op):
    p, ins, x = _one(E, 'spatial_padding', (2, 4, 5, 3), lambda X: op.spatial_padding(X, [1, 2], [0, 3]))
    return p, ins, np.pad(x, ((0, 0), (1, 0), (2, 3), (0, 0))), True


def flip(E, op):
    p, ins, x = _one(E, 'flip', (3, 4, 5), lambda X: op.flip(X, [0, 2]))
    return p, ins, np.flip(x, (0, 2)), True


def repeat(E, op):
    p, ins, x = _one(E, 'repeat', (2, 3, 4), lambda X: op.repeat(X, 3, 1))
    return p, ins, np.repeat(x, 3, 1), True


def tile(E, op):
    p, ins, x = _one(E, 'tile', (2, 3, 4), lambda X: op.tile(X, [2, 1, 3]))
    return p, ins, np.tile(x, (2, 1, 3)), True


def transpose(E, op):
    p, ins, x = _one(E, 'transpose', (2, 3, 4, 5), lambda X: op.transpose(X, [0, 3, 1, 2]))
    return p, ins, np.transpose(x, (0, 3, 1, 2)), True


def transpose_default(E, op):
    p, ins, x = _one(E, 'transpose', (6, 7), lambda X: op.transpose(X))
    return p, ins, x.T, True


def reshape(E, op):
    p, ins, x = _one(E, 'reshape', (2, 3, 4), lambda X: op.reshape(X, [0, -1]))  # keep dim 0, infer the rest
    return p, ins, x.reshape(2, 12), True


def squeeze_unsqueeze(E, op):
    p, ins, x = _one(E, 'squeeze', (2, 1, 3, 1), lambda X: op.unsqueeze(op.squeeze(X, [1, 3]), [0]))
    return p, ins, x.reshape(1, 2, 3), True


def prod(E, op):
    p, ins, x = _one(E, 'prod', (3, 4, 5), lambda X: op.prod(X, [1], True))
    return p, ins, np.prod(x.astype(np.float64), 1, keepdims=True), False


def variance(E, op):
    p, ins, x = _one(E, 'variance', (4, 6, 5), lambda X: op.variance(X, [0, 2]))
    return p, ins, np.var(x.astype(np.float64), (0, 2)), False


def arithmetic(E, op):
    """abs, square, sigmoid, elu, hard_sigmoid on one input, summed with distinct weights."""
    X = _f32(E, (5, 7))
    x = (_rng().standard_normal((5, 7)) * 3).astype(np.float32)
    O = op.abs(X) + 2 * op.square(X) + 4 * op.sigmoid(X) + 8 * op.elu(X, 0.5) + 16 * op.hard_sigmoid(X, 0.2)
    x64 = x.astype(np.float64)
    ref = (np.abs(x64) + 2 * x64 * x64 + 4 / (1 + np.exp(-x64)) + 8 * np.where(x64 < 0, 0.5 * np.exp(x64) - 0.5, x64) +
           16 * np.clip(0.2 * x64 + 0.5, 0, 1))
    return E.Program('arithmetic', [X], [O]), [x], ref, False


def _broadcast_ref(E, op, in_shape, data, rshape, axes, expected):
    X = _f32(E, in_shape)
    x = np.asarray(data, np.float32).reshape(in_shape)
    return E.Program('broadcast', [X], [op.broadcast(X, rshape, axes)]), [x], np.asarray(expected, np.float32).reshape(rshape), True


def broadcast_noop_reference(E, op):
    return _broadcast_ref(E, op, (3,), [0, 1, 2], [3], [0], [0, 1, 2])


def broadcast_scalar_reference(E, op):
    return _broadcast_ref(E, op, (), [3], [3, 4], [], [3] * 12)


def broadcast_noop_large_reference(E, op):
    return _broadcast_ref(E, op, (3, 4), [0, 1, 2, 3] * 3, [3, 4], [0, 1], [0, 1, 2, 3] * 3)


def broadcast_numpy_reference(E, op):
    return _broadcast_ref(E, op, (1, 3, 3), [0, 1, 2] * 3, [1, 4, 3, 3], [0, 2, 3], [0, 1, 2] * 12)


def broadcast_numpy2_reference(E, op):
    return _broadcast_ref(E, op, (3, 1), [0, 1, 2], [3, 4], [0, 1], [0] * 4 + [1] * 4 + [2] * 4)


def broadcast_numpy3_reference(E, op):
    return _broadcast_ref(E, op, (3,), [0, 1, 2], [4, 3], [1], [0, 1, 2] * 4)


def broadcast_non_numpy_reference(E, op):
    return _broadcast_ref(E, op, (3,), [0, 1, 2], [3, 4], [0], [0] * 4 + [1] * 4 + [2] * 4)


def _reorg_yolo_ref(x, stride, decrease):
    """What the reference's test expects (its loop nest, plaidml/op/op_test.cc:524-550, in closed form), NCHW:
    channel k = off * C_small + c of the wide tensor holds pixel (oy, ox) = (off / s, off % s) of every s x s block
    of channel c of the spatially large tensor.  decrease: wide -> large; otherwise large -> wide."""
    s_ = stride
    if decrease:
        n, c, h, w = x.shape
        cs = c // (s_ * s_)
        return x.reshape(n, s_, s_, cs, h, w).transpose(0, 3, 4, 1, 5, 2).reshape(n, cs, h * s_, w * s_)
    n, c, h, w = x.shape
    return x.reshape(n, c, h // s_, s_, w // s_, s_).transpose(0, 3, 5, 1, 2, 4).reshape(n, c * s_ * s_, h // s_, w // s_)


def _reorg(E, op, decrease):
    N, C, H, W, S = 1, 4, 6, 6, 2
    X = E.Placeholder(E.DType.INT64, [N, C, H, W])
    x = np.arange(N * C * H * W, dtype=np.int64).reshape(N, C, H, W)
    return E.Program('reorg_yolo', [X], [op.reorg_yolo(X, S, decrease)]), [x], _reorg_yolo_ref(x, S, decrease), True


def reorg_yolo_decrease_reference(E, op):
    return _reorg(E, op, True)


def reorg_yolo_increase_reference(E, op):
    return _reorg(E, op, False)


def reorg_yolo_nhwc(E, op):
    """The NHWC lens: the same rearrangement as NCHW on the transposed tensor."""
    N, C, H, W, S = 2, 8, 4, 6, 2
    X = E.Placeholder(E.DType.FLOAT32, [N, H, W, C])
    x = _rng().standard_normal((N, H, W, C)).astype(np.float32)
    ref = _reorg_yolo_ref(x.transpose(0, 3, 1, 2), S, False).transpose(0, 2, 3, 1)
    return E.Program('reorg_yolo', [X], [op.reorg_yolo(X, S, False, 'NHWC')]), [x], ref, True


def all_any(E, op):
    X = E.Placeholder(E.DType.INT32, [3, 4, 5])
    x = _rng().integers(-1, 2, (3, 4, 5)).astype(np.int32)
    x[1] = np.abs(x[1]) + 1
    outs = [op.all(X, [1]), op.any(X, [0, 2], True), op.all(X), op.any(X, [])]
    ref = [x.all(1).astype(np.uint8), x.any((0, 2), keepdims=True).astype(np.uint8), np.uint8(x.all()), (x != 0).astype(np.uint8)]
    return E.Program('all_any', [X], outs), [x], ref, True


def binary_crossentropy(E, op):
    T, P = _f32(E, (4, 6)), _f32(E, (4, 6))
    r = _rng()
    t = r.integers(0, 2, (4, 6)).astype(np.float32)
    p = r.uniform(-0.1, 1.1, (4, 6)).astype(np.float32)
    pc = np.clip(p.astype(np.float64), 0.01, 0.99)
    ref = -t * np.log(pc) - (1 - t) * np.log(1 - pc)
    return E.Program('bce', [T, P], [op.binary_crossentropy(T, P, 0.01)]), [t, p], ref, False


def cumprod(E, op):
    p, ins, x = _one(E, 'cumprod', (3, 6, 4), lambda X: op.cumprod(X, 1))
    return p, ins, np.cumprod(x.astype(np.float64), 1), False


def l2norm(E, op):
    X = _f32(E, (3, 5, 4))
    x = _rng().standard_normal((3, 5, 4)).astype(np.float32)
    x[1] = 0
    x64 = x.astype(np.float64)
    ss = (x64 * x64).sum((1, 2), keepdims=True)
    outs = [op.l2norm(X, [1, 2], 0.25, op.EPS_ADD), op.l2norm(X, [1, 2], 0.25, op.EPS_MAX)]
    return E.Program('l2norm', [X], outs), [x], [np.sqrt(ss + 0.25), np.sqrt(np.maximum(ss, 0.25))], False


def lrn(E, op):
    """Across-channel normalisation, window 5 (AlexNet's), against the explicit window sum; an even window
    too, which reaches one element further back than forward (offsets -w/2 .. w - 1 - w/2)."""
    X = _f32(E, (2, 3, 4, 9))
    x = _rng().standard_normal((2, 3, 4, 9)).astype(np.float32)
    x64 = x.astype(np.float64)

    def ref(w, alpha, beta, eps):
        sq = np.zeros_like(x64)
        for c in range(9):
            lo, hi = c - w // 2, c + w - 1 - w // 2
            sq[..., c] = (x64[..., max(lo, 0):min(hi, 8) + 1] ** 2).sum(-1)
        return x64 / (alpha * sq + eps) ** beta

    outs = [op.lrn(X, [5], (-1,), 1e-2, 0.75, 2.0), op.lrn(X, [4], (3,), 0.5, 0.5, 1.0)]
    return E.Program('lrn', [X], outs), [x], [ref(5, 1e-2, 0.75, 2.0), ref(4, 0.5, 0.5, 1.0)], False


def mvn(E, op):
    X = _f32(E, (2, 5, 4, 3))
    x = _rng().standard_normal((2, 5, 4, 3)).astype(np.float32) * 3 + 1
    x64 = x.astype(np.float64)
    m = x64.mean((1, 2), keepdims=True)
    sd = x64.std((1, 2), keepdims=True)
    m2 = x64.mean((1, 2, 3), keepdims=True)
    outs = [op.mvn(X, layout='NHWC', across_channels=False), op.mvn(X, axes=[1, 2, 3], normalize_variance=False)]
    return E.Program('mvn', [X], outs), [x], [(x64 - m) / np.maximum(sd, 1e-9), x64 - m2], False


def slice_of(E, op):
    X = _f32(E, (6, 7, 5))
    x = _rng().standard_normal((6, 7, 5)).astype(np.float32)
    outs = [op.slice_of(X, [slice(1, 5, 2), 3, slice(None, None, None)]),
            op.slice_of(X, [slice(None, None, -1), slice(-3, None, None), -1]),
            op.slice_of(X, [slice(4, 0, -2), slice(None, -2, 3), slice(1, 2, None)])]
    ref = [x[1:5:2, 3, :], x[::-1, -3:, -1], x[4:0:-2, :-2:3, 1:2]]
    return E.Program('slice', [X], outs), [x], ref, True


def scale_gradient(E, op):
    p, ins, x = _one(E, 'scale_gradient', (3, 4), lambda X: op.scale_gradient(X, 0.5) + 0.0)
    return p, ins, x, True


def sort_reference(E, op):
    """OpTest.Sort, plaidml/op/op_test.cc:638-658."""
    data = [81.69, 95.74, 27.74, 43.69, 55.79, 56.79, 57.52, 5.9, 39.48, 7.11, 14.81, 66.23, 20.25, 66.05, 64.5, 71.07, 67.6,
            54.42, 87.59, 80.02]
    want = [27.74, 43.69, 81.69, 95.74, 5.9, 55.79, 56.79, 57.52, 7.11, 14.81, 39.48, 66.23, 20.25, 64.5, 66.05, 71.07, 54.42,
            67.6, 80.02, 87.59]
    p, ins, _ = _one(E, 'sort', (5, 4), lambda X: op.sort(X, 1, E.SORT_ASC), data)
    return p, ins, np.array(want, np.float32).reshape(5, 4), True


def sort_descending_axis0(E, op):
    p, ins, x = _one(E, 'sort', (6, 3, 4), lambda X: op.sort(X, 0, E.SORT_DESC))
    return p, ins, -np.sort(-x, axis=0), True


def gather_nd_reference(E, op):
    """CppEdsl.GatherND / GatherNDWithBatchDims, plaidml/edsl/tests/edsl_test.cc:1661-1710."""
    A, B = _f32(E, (2, 2, 2)), E.Placeholder(E.DType.INT32, [2, 2])
    C, D = _f32(E, (2, 3, 4)), E.Placeholder(E.DType.INT32, [2, 3, 1, 1])
    prog = E.Program('gatherND', [A, B, C, D], [op.gatherND(A, B), op.gatherND(C, D, batch_dims=2)])
    ins = [np.array([-5, -6, 1.3, 4.5, -7, 4, 5, 6], np.float32).reshape(2, 2, 2), np.array([0, 1, 1, 0], np.int32).reshape(2, 2),
           np.arange(1, 25, dtype=np.float32).reshape(2, 3, 4), np.array([1, 0, 2, 0, 2, 2], np.int32).reshape(2, 3, 1, 1)]
    return prog, ins, [np.array([1.3, 4.5, -7, 4], np.float32).reshape(2, 2),
                       np.array([2, 5, 11, 13, 19, 23], np.float32).reshape(2, 3, 1)], True


def gather_nd_linear_reference(E, op):
    """CppEdsl.InterpolatedGatherND1 / ND2 / ND3, plaidml/edsl/tests/edsl_test.cc:1712-1794."""
    A, B1, B3 = _f32(E, (2, 2)), _f32(E, (3, 1)), _f32(E, (3, 2))
    C, B2 = _f32(E, (4, 3, 2)), _f32(E, (4, 1, 2))
    lin = E.INTERP_LINEAR
    prog = E.Program('gatherND', [A, B1, B3, C, B2],
                     [op.gatherND(A, B1, interpolation_mode=lin), op.gatherND(C, B2, batch_dims=1, interpolation_mode=lin),
                      op.gatherND(A, B3, interpolation_mode=lin)])
    a = np.array([-5, -6, 1.3, 4.5], np.float32).reshape(2, 2)
    c = np.array([-5, -6, 1.3, 4.5, 2, 3.5, 0.3, 4.1, -5, 6, 1.1, 0.5, 1, 2, 3, 4, 5, 6, 0.8, 0.5, 2, -6, 1.9, 9.5],
                 np.float32).reshape(4, 3, 2)
    ins = [a, np.array([0.2, 0.5, 0.9], np.float32).reshape(3, 1), np.array([0.2, 0.5, 0.3, 0.9, 0.5, 0.5], np.float32).reshape(3, 2),
           c, np.array([0.2, 0.5, 0.2, 0.9, 0.2, 0.5, 0.2, 0.9], np.float32).reshape(4, 1, 2)]
    want = [np.array([-3.74, -3.9, -1.85, -0.75, 0.67, 3.45], np.float32).reshape(3, 2),
            np.array([-3.82, 3.956, 1.9, -0.616], np.float32).reshape(4, 1),
            np.array([-3.82, -2.876, -1.3], np.float32)]
    return prog, ins, want, False


def topk(E, op):
    X = _f32(E, (4, 9))
    x = _rng().standard_normal((4, 9)).astype(np.float32)
    v, i = op.topk(X, 3, axis=1)                                              # largest three, by value
    v2, i2 = op.topk(X, 4, axis=1, sort_direction=E.SORT_ASC, sort_type=op.TOPK_INDEX)   # smallest four, in position order
    order = np.argsort(-x, axis=1, kind='stable')[:, :3]
    small = np.sort(np.argsort(x, axis=1, kind='stable')[:, :4], axis=1)
    want = [np.take_along_axis(x, order, 1), order.astype(np.int32), np.take_along_axis(x, small, 1), small.astype(np.int32)]
    return E.Program('topk', [X], [v, i, v2, i2]), [x], want, True


def _tent_resize(x, fh, fw):
    """Every input pixel spread over the output with the separable tent weights 1 - |d| / f at offsets |d| < f
    around f * position (direct accumulation; float64)."""
    n, h, w, c = x.shape
    out = np.zeros((n, fh * h, fw * w, c))
    for a in range(h):
        for b in range(w):
            for dy in range(-fh + 1, fh):
                for dx in range(-fw + 1, fw):
                    oy, ox = fh * a + dy, fw * b + dx
                    if 0 <= oy < fh * h and 0 <= ox < fw * w:
                        out[:, oy, ox, :] += x[:, a, b, :] * (1 - abs(dy) / fh) * (1 - abs(dx) / fw)
    return out


def image_resize(E, op):
    X = _f32(E, (2, 4, 5, 3))
    x = _rng().standard_normal((2, 4, 5, 3)).astype(np.float32)
    Xc = _f32(E, (2, 3, 4, 5))
    outs = [op.image_resize(X, [2, 3], op.RESIZE_NEAREST), op.image_resize(X, [3, 2], op.RESIZE_BILINEAR),
            op.image_resize(Xc, [2, 2], op.RESIZE_BILINEAR, op.LAYOUT_NCX)]
    xc = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    want = [np.repeat(np.repeat(x, 2, 1), 3, 2), _tent_resize(x.astype(np.float64), 3, 2),
            _tent_resize(x.astype(np.float64), 2, 2).transpose(0, 3, 1, 2)]
    return E.Program('image_resize', [X, Xc], outs), [x, xc], want, False


CASES = {f.__name__: f for f in (
    image_resize,
    sort_reference, sort_descending_axis0, gather_nd_reference, gather_nd_linear_reference, topk,
    broadcast_noop_reference, broadcast_scalar_reference, broadcast_noop_large_reference, broadcast_numpy_reference,
    broadcast_numpy2_reference, broadcast_numpy3_reference, broadcast_non_numpy_reference, reorg_yolo_decrease_reference,
    reorg_yolo_increase_reference, reorg_yolo_nhwc, all_any, binary_crossentropy, cumprod, l2norm, lrn, mvn, slice_of,
    scale_gradient,
    concatenate, cumsum, cumsum_exclusive_reference, explicit_padding_reference, explicit_padding_neg_inf_reference,
    explicit_padding_inf_reference, explicit_padding_noop_reference, explicit_padding_edge_reference, spatial_padding, flip,
    repeat, tile, transpose, transpose_default, reshape, squeeze_unsqueeze, prod, variance, arithmetic)}

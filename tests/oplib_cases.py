"""Cases for the data-movement / simple-arithmetic operations of the op library, each built twice (oracle
and product EDSL): name -> builder(E, op) returning (program, inputs, expected numpy result, exact?).

Expected values are numpy closed forms (np.concatenate, np.pad, np.cumsum, ...) and, where the reference holds
an exact case, that case (plaidml/op/op_test.cc: CumSumExclusive :297-304, ExplicitPadding :318-333,
ExplicitPaddingNegInf :335-351, ExplicitPaddingInf :353-370, ExplicitPaddingNoOp :372-383,
ExplicitPaddingEdge :385-418).
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


CASES = {f.__name__: f for f in (
    concatenate, cumsum, cumsum_exclusive_reference, explicit_padding_reference, explicit_padding_neg_inf_reference,
    explicit_padding_inf_reference, explicit_padding_noop_reference, explicit_padding_edge_reference, spatial_padding, flip,
    repeat, tile, transpose, transpose_default, reshape, squeeze_unsqueeze, prod, variance, arithmetic)}

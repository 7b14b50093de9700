"""Small whole-program cases with the answers the reference's tests hold (plaidml/edsl/tests/edsl_test.cc; the
TEST_F line with each): constants as operands, mixed signedness, literals on the left, reshapes to and from
scalars.  A case is build(E) -> (inputs, outputs), input arrays, expected arrays (compared bit-exactly)."""
import numpy as np


def _p(E, dt, shape):
    return E.Placeholder(getattr(E.DType, dt), list(shape))


def simple_add(E):            # :124
    A, B = _p(E, 'FLOAT32', (3, 3)), _p(E, 'FLOAT32', (3, 3))
    x = np.arange(1, 10, dtype=np.float32).reshape(3, 3)
    return [A, B], [A + B], [x, x], [2 * x]


def const_add(E):             # :376  two constants, no inputs
    A = E.Constant(np.array([4, 3, 2, 1], np.int32), name='A')
    B = E.Constant(np.array([1, 2, 3, 4], np.int32), name='B')
    return [], [A + B], [], [np.array([5, 5, 5, 5], np.int32)]


def mixed_add(E):             # :396  (si32 constant + si32 constant) + ui32 input -> ui32
    I = _p(E, 'UINT32', (4,))
    A = E.Constant(np.array([4, 3, 2, 1], np.int32), name='A')
    B = E.Constant(np.array([1, 2, 3, 4], np.int32), name='B')
    return [I], [(A + B) + I], [np.array([1, 2, 2, 1], np.uint32)], [np.array([6, 7, 7, 6], np.uint32)]


def reciprocal(E):            # :981
    A = _p(E, 'FLOAT32', (6,))
    return [A], [1.0 / A], [np.array([1, 2, 4, 5, 8, 10], np.float32)], [np.array([1.0, 0.5, 0.25, 0.2, 0.125, 0.1], np.float32)]


def reshape_fold(E):          # :997
    A = _p(E, 'INT32', (3, 3))
    x = np.arange(1, 10, dtype=np.int32).reshape(3, 3)
    return [A], [E.reshape(A, [3, 3])], [x], [x]


def reshape_scalar(E):        # :1015
    A = _p(E, 'INT32', ())
    return [A], [E.reshape(A, [])], [np.array(2, np.int32)], [np.array(2, np.int32)]


def reshape_into_scalar(E):   # :1030
    A = _p(E, 'INT32', (1, 1, 1))
    return [A], [E.reshape(A, [])], [np.array([[[2]]], np.int32)], [np.array(2, np.int32)]


def reshape_from_scalar(E):   # :1047
    A = _p(E, 'INT32', ())
    return [A], [E.reshape(A, [1, 1, 1])], [np.array(2, np.int32)], [np.array([[[2]]], np.int32)]


CASES = {f.__name__: f for f in (simple_add, const_add, mixed_add, reciprocal, reshape_fold, reshape_scalar, reshape_into_scalar,
                                 reshape_from_scalar)}


def run_case(name, E, **kw):
    ins, outs, arrays, expected = CASES[name](E)
    got = E.run(E.Program(name, ins, outs), arrays, **kw)
    assert len(got) == len(expected)
    for g, e in zip(got, expected):
        assert g.shape == e.shape and g.dtype == e.dtype, (name, g.shape, g.dtype, e.shape, e.dtype)
        np.testing.assert_array_equal(g, e, err_msg=name)

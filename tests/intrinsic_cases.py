"""Elementwise intrinsics with the answers the reference's own tests hold for them
(plaidml/edsl/tests/edsl_test.cc; line numbers with each case).  Every case is
(build(E) -> (inputs, output), input arrays, expected array, tolerance) where tolerance None means
bit-exact and a number t means |x - y| <= (|x| + |y|) * t, the reference fixture's rule
(plaidml/testenv.cc:53-67)."""
import numpy as np

U64, I32, F32, U8 = 'UINT64', 'INT32', 'FLOAT32', 'UINT8'
_NP = {U64: np.uint64, I32: np.int32, F32: np.float32, U8: np.uint8}

_ONE_TO_NINE = [1, 2, 3, 4, 5, 6, 7, 8, 9]
_TEN_UP = [10, 11, 12, 13, 14, 15, 16, 17, 18]
_SHIFTED = [k << (9 + k) for k in _ONE_TO_NINE]
_HOLES = [1, 2, 3, 4, 0, 6, 7, 0, 9]
_UNIT = [0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 1.0, 0.0, -0.6]


def _case(line, dtypes, fn, inputs, expected, tol=None, out=None):
    def build(E):
        ins = [E.Placeholder(getattr(E.DType, d), [3, 3]) for d in dtypes]
        return ins, fn(E, *ins)
    arrays = [np.array(v, _NP[d]).reshape(3, 3) for v, d in zip(inputs, dtypes)]
    exp = np.array(expected, out if out is not None else _NP[dtypes[0]]).reshape(3, 3)
    return dict(line=line, build=build, inputs=arrays, expected=exp, tol=tol)


CASES = {
    'bit_and_scalar': _case(180, [U64], lambda E, a: a & 0xFFFFFFFF,
                            [[(1 << (32 + k)) + k for k in range(9)]], list(range(9))),
    'bit_and': _case(197, [U64, U64], lambda E, a, b: a & b, [_ONE_TO_NINE, _TEN_UP],
                     [x & y for x, y in zip(_ONE_TO_NINE, _TEN_UP)]),
    'bit_or': _case(215, [U64, U64], lambda E, a, b: a | b, [_ONE_TO_NINE, _TEN_UP],
                    [x | y for x, y in zip(_ONE_TO_NINE, _TEN_UP)]),
    'bit_left': _case(233, [U64, U64], lambda E, a, b: a << b, [_ONE_TO_NINE, _TEN_UP], _SHIFTED),
    'bit_right_tensor': _case(255, [U64, U64], lambda E, a, b: a >> b, [_SHIFTED, _TEN_UP], _ONE_TO_NINE),
    'bit_right_scalar': _case(273, [U64], lambda E, a: a >> 9, [_SHIFTED], [k << k for k in _ONE_TO_NINE]),
    'bit_not': _case(289, [U8], lambda E, a: ~a, [[0x00, 0x01, 0x02, 0x10, 0x11, 0x22, 0xF0, 0x0F, 0xFF]],
                     [0xFF, 0xFE, 0xFD, 0xEF, 0xEE, 0xDD, 0x0F, 0xF0, 0x00]),
    'bit_xor': _case(304, [U64, U64], lambda E, a, b: a ^ b, [_ONE_TO_NINE, _TEN_UP],
                     [x ^ y for x, y in zip(_ONE_TO_NINE, _TEN_UP)]),
    'mod': _case(606, [I32, I32], lambda E, a, b: a % b, [[2, 4, 8, 16, 32, 64, 128, 256, 512], _ONE_TO_NINE],
                 [2 % 1, 4 % 2, 8 % 3, 16 % 4, 32 % 5, 64 % 6, 128 % 7, 256 % 8, 512 % 9]),
    'cos': _case(1162, [F32], lambda E, a: E.cos(a), [[5, 6, 7, 4, 5, 6, 7, 8, 9]],
                 [0.283662, 0.96017, 0.753902, -0.653644, 0.283662, 0.96017, 0.753902, -0.1455, -0.91113], 1e-4),
    'sin': _case(1177, [F32], lambda E, a: E.sin(a), [[5, 6, 7, 4, -5, 1.1, 7, 8, 9]],
                 [-0.958924, -0.279415, 0.656987, -0.756802, 0.958924, 0.891207, 0.656987, 0.989358, 0.412118], 1e-4),
    'logical_and_uint64': _case(1203, [U64, U64], lambda E, a, b: E.logical_and(a, b), [_HOLES, _TEN_UP],
                                [1, 1, 1, 1, 0, 1, 1, 0, 1], out=np.bool_),
    'logical_and_mixed': _case(1223, [U64, F32], lambda E, a, b: E.logical_and(a, b), [_HOLES, _TEN_UP],
                               [1, 1, 1, 1, 0, 1, 1, 0, 1], out=np.bool_),
    'logical_or_uint64': _case(1243, [U64, U64], lambda E, a, b: E.logical_or(a, b),
                               [_HOLES, [10, 11, 12, 0, 0, 0, 16, 17, 18]], [1, 1, 1, 1, 0, 1, 1, 1, 1], out=np.bool_),
    'logical_or_float': _case(1264, [F32, F32], lambda E, a, b: E.logical_or(a, b),
                              [_HOLES, [10, 11, 12, 0, 0, 0, 16, 17, 18]], [1, 1, 1, 1, 0, 1, 1, 1, 1], out=np.bool_),
    'logical_or_int32': _case(1282, [I32, I32], lambda E, a, b: E.logical_or(a, b),
                              [_HOLES, [10, 11, 12, 0, 0, 0, 16, 17, 18]], [1, 1, 1, 1, 0, 1, 1, 1, 1], out=np.bool_),
    'logical_not_int32': _case(1300, [I32], lambda E, a: E.logical_not(a), [_HOLES],
                               [0, 0, 0, 0, 1, 0, 0, 1, 0], out=np.bool_),
    'logical_not_float': _case(1315, [F32], lambda E, a: E.logical_not(a), [[1.0, 2.0, 3.0, 4.0, 0, 6.5, 7.7, 0, 0.9]],
                               [0, 0, 0, 0, 1, 0, 0, 1, 0], out=np.bool_),
    'asin': _case(1330, [F32], lambda E, a: E.asin(a), [_UNIT],
                  [0.100167, 0.201358, 0.304693, 0.411517, 0.523599, 0.643501, 1.5708, 0.0, -0.643501], 1e-5),
    'asinh': _case(1349, [F32], lambda E, a: E.asinh(a), [_UNIT],
                   [0.099834, 0.198690, 0.295673, 0.390035, 0.481212, 0.568825, 0.881374, 0.0, -0.568826], 1e-5),
    'acos': _case(1368, [F32], lambda E, a: E.acos(a), [_UNIT],
                  [1.47063, 1.36944, 1.2661, 1.15928, 1.0472, 0.927295, 0.0, 1.5708, 2.2143], 1e-4),
    'acosh': _case(1387, [F32], lambda E, a: E.acosh(a), [[1.1, 1.2, 1.3, 1.4, 1.5, 1.6, 1.7, 1.8, 1.0]],
                   [0.443568, 0.622363, 0.756433, 0.867015, 0.962424, 1.04697, 1.12323, 1.19291, 0.0], 1e-4),
    'atan': _case(1406, [F32], lambda E, a: E.atan(a), [_UNIT],
                  [0.0996687, 0.197396, 0.291457, 0.380506, 0.463648, 0.54042, 0.785398, 0, -0.54042], 1e-5),
    'atanh': _case(1425, [F32], lambda E, a: E.atanh(a), [[0.1, 0.2, 0.3, 0.4, 0.5, 0.6, 0.0, -0.3, -0.6]],
                   [0.100335, 0.202733, 0.30952, 0.423649, 0.549306, 0.693147, 0., -0.30952, -0.693147], 1e-5),
    'cosh': _case(1444, [F32], lambda E, a: E.cosh(a), [_UNIT],
                  [1.005, 1.02007, 1.04534, 1.08107, 1.12763, 1.18547, 1.54308, 1, 1.18547], 1e-5),
    'erf': _case(1463, [F32], lambda E, a: E.erf(a), [_UNIT],
                 [0.112463, 0.222703, 0.328627, 0.428392, 0.5205, 0.603856, 0.842701, 0, -0.603856], 1e-5),
    'floor': _case(1482, [F32], lambda E, a: E.floor(a), [[1.1, 9.21, 3.0, -0.4, -7.0, 0.6, 1.0, 0.0, -6.6]],
                   [1, 9, 3, -1, -7, 0, 1, 0, -7]),
    'pow': _case(1796, [F32, F32], lambda E, a, b: E.pow(a, b), [[0.5, 1.5, 2.5] * 3, [0.5] * 3 + [1.5] * 3 + [2.5] * 3],
                 [0.707107, 1.22474, 1.58114, 0.353553, 1.83712, 3.95285, 0.176777, 2.75568, 9.88212], 1e-5),
    'round': _case(1819, [F32], lambda E, a: E.round(a), [[1.1, 9.21, 3.0, -0.4, -7.0, 0.6, 1.0, 0.0, -6.6]],
                   [1, 9, 3, -0., -7, 1, 1, 0, -7]),
    'sinh': _case(1838, [F32], lambda E, a: E.sinh(a), [[-2.0, -1.5, 0.0, -1.0, 0.1, 0.2, 1.0, 1.5, 5.0]],
                  [-3.62686, -2.12928, 0, -1.1752, 0.100167, 0.201336, 1.1752, 2.12928, 74.2032], 1e-5),
    'tan': _case(1857, [F32], lambda E, a: E.tan(a), [_UNIT],
                 [0.100335, 0.20271, 0.309336, 0.422793, 0.546302, 0.684137, 1.55741, 0, -0.684137], 1e-4),
}


def check_case(name, got):
    c = CASES[name]
    exp = c['expected']
    assert got.shape == exp.shape and got.dtype == exp.dtype, (name, got.dtype, exp.dtype)
    if c['tol'] is None:
        np.testing.assert_array_equal(got, exp, err_msg=name)
    else:
        g, e = got.astype(np.float64), exp.astype(np.float64)
        # the reference's expected values are printed with six significant digits
        bound = (np.abs(g) + np.abs(e)) * c['tol'] + 1e-6
        assert (np.abs(g - e) <= bound).all(), (name, got, exp)


def run_case(name, E):
    c = CASES[name]
    ins, out = c['build'](E)
    return E.run(E.Program(name, ins, [out]), c['inputs'])[0]

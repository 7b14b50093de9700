"""argsort / gather / scatter with the answers the reference's own tests hold (plaidml/edsl/tests/edsl_test.cc;
the line of each TEST_F is given with the case).  A case is (build(E) -> (inputs, output), input arrays, expected,
tolerance): tolerance None = bit-exact, a number t = |x - y| <= (|x| + |y|) * t (plaidml/testenv.cc:53-67)."""
import numpy as np

F32, F64, F16, I32 = 'FLOAT32', 'FLOAT64', 'FLOAT16', 'INT32'
_NP = {F32: np.float32, F64: np.float64, F16: np.float16, I32: np.int32}


def _case(line, specs, fn, inputs, expected, tol=None, out_dtype=None):
    def build(E):
        ins = [E.Placeholder(getattr(E.DType, d), list(shape)) for d, shape in specs]
        return ins, fn(E, *ins)
    arrays = [np.array(v, _NP[d]).reshape(shape) for v, (d, shape) in zip(inputs, specs)]
    exp = np.array(expected, out_dtype if out_dtype is not None else _NP[specs[0][0]])
    return dict(line=line, build=build, inputs=arrays, expected=exp, tol=tol)


_SIX = [0.0, 1.0, 8.0, 5.0, 5.0, 2.0]
_POS12 = [-0.25, 0.25, 0.75, 1.25, 1.75, 2.25, 2.75, 3.25, 3.75, 4.25, 4.75, 5.25]
_CUBIC = [-0.0703125, 0.0390625, 0.304688, 2.5625, 6.8125, 7.88281, 5.77344, 4.85938, 5.14062, 4.39062, 2.60938, 1.78906]
_A3 = [[v + k / 10 for v in range(1, 11)] for k in range(3)]   # 3 x 5 x 2: 1..10, 1.1..10.1, 1.2..10.2
_Z64, _O64 = [0.0] * 64, [1.0] * 64
_U32 = [5] * 4 + [6] * 4 + [7] * 4 + [8] * 4
_SORT20 = [81.69, 95.74, 27.74, 43.69, 55.79, 56.79, 57.52, 5.9, 39.48, 7.11, 14.81, 66.23, 20.25, 66.05, 64.5, 71.07, 67.6,
           54.42, 87.59, 80.02]
_ORDER20 = [7, 9, 10, 12, 2, 8, 3, 17, 4, 5, 6, 14, 13, 11, 16, 15, 19, 0, 18, 1]


def _rows(values, where):
    out = list(values)
    for at, row in where:
        out[at * 16:(at + 1) * 16] = row
    return out


CASES = {
    'gather': _case(1490, [(F32, (3, 2)), (I32, (4,))], lambda E, a, b: E.gather(a, b, axis=1),
                    [[-5, -6, -7, 4, 5, 6], [0, 1, 1, 0]], np.array([-5, -6, -6, -5, -7, 4, 4, -7, 5, 6, 6, 5]).reshape(3, 4)),
    'gather_nearest_prefer_ceil': _case(
        1510, [(F32, (1, 6)), (F32, (9,))],
        lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_NEAREST, nearest_mode=E.NEAREST_ROUND_PREFER_CEIL),
        [[0.3, 1.0, 8.0, 5.0, 5.0, 2.0], [-0.25, 0.5, 0.75, 1.5, 2.0, 5.0, 5.1, 5.5, 5.6]],
        np.array([0.3, 1.0, 1.0, 8.0, 8.0, 2.0, 2.0, 2.0, 2.0]).reshape(1, 9)),
    'gather_linear': _case(1523, [(F32, (1, 6)), (F32, (12,))],
                           lambda E, a, b: E.gather(a, b, axis=-1, interpolation_mode=E.INTERP_LINEAR), [_SIX, _POS12],
                           np.array([0.0, 0.25, 0.75, 2.75, 6.25, 7.25, 5.75, 5.0, 5.0, 4.25, 2.75, 2.0]).reshape(1, 12)),
    'gather_linear_return_zero': _case(
        1535, [(F32, (1, 6)), (F32, (12,))],
        lambda E, a, b: E.gather(a, b, axis=-1, interpolation_mode=E.INTERP_LINEAR, out_of_bounds_mode=E.OOB_RETURN_ZERO),
        [_SIX, _POS12], np.array([0.0, 0.25, 0.75, 2.75, 6.25, 7.25, 5.75, 5.0, 5.0, 4.25, 2.75, 0.0]).reshape(1, 12)),
    'gather_cubic': _case(1548, [(F32, (1, 6)), (F32, (12,))],
                          lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_CUBIC, cube_coeff=-0.5),
                          [_SIX, _POS12], np.array(_CUBIC).reshape(1, 12), 1e-5),
    'gather_cubic_return_zero': _case(
        1561, [(F32, (1, 6)), (F32, (12,))],
        lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_CUBIC, cube_coeff=-0.5,
                                 out_of_bounds_mode=E.OOB_RETURN_ZERO),
        [_SIX, _POS12], np.array([0.0] + _CUBIC[1:-1] + [0.0]).reshape(1, 12), 1e-5),
    'gather_cubic_double': _case(1578, [(F64, (1, 6)), (F64, (12,))],
                                 lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_CUBIC, cube_coeff=-0.5),
                                 [_SIX, _POS12], np.array(_CUBIC).reshape(1, 12), 1e-5),
    'gather_cubic_half': _case(1591, [(F16, (1, 6)), (F16, (12,))],
                               lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_CUBIC, cube_coeff=-0.5),
                               [_SIX, _POS12], np.array(_CUBIC).reshape(1, 12), 1e-2),
    'gather_nearest_multi_d_indices': _case(
        1617, [(F32, (3, 5, 2)), (F32, (2, 2))], lambda E, a, b: E.gather(a, b, axis=1, interpolation_mode=E.INTERP_NEAREST),
        [_A3, [0.8, 1.3, 2.0, 2.7]],
        np.array([[[3 + k / 10, 4 + k / 10], [3 + k / 10, 4 + k / 10], [5 + k / 10, 6 + k / 10], [7 + k / 10, 8 + k / 10]]
                  for k in range(3)]).reshape(3, 2, 2, 2)),
    'gather_nd': _case(1661, [(F32, (2, 2, 2)), (I32, (2, 2))], lambda E, a, b: E.gather(a, b, mode=E.GATHER_ND),
                       [[-5, -6, 1.3, 4.5, -7, 4, 5, 6], [0, 1, 1, 0]], np.array([1.3, 4.5, -7, 4]).reshape(2, 2)),
    'gather_nd_batch_dims': _case(1682, [(F32, (2, 3, 4)), (I32, (2, 3, 1, 1))],
                                  lambda E, a, b: E.gather(a, b, mode=E.GATHER_ND, batch_dims=2),
                                  [list(range(1, 25)), [1, 0, 2, 0, 2, 2]], np.array([2, 5, 11, 13, 19, 23]).reshape(2, 3, 1)),
    'scatter_1d': _case(1874, [(F32, (8,)), (I32, (4,)), (F32, (4,))], lambda E, d, i, u: E.scatter(d, i, u),
                        [[0] * 8, [4, 3, 1, 7], [9, 10, 11, 12]], [0, 11, 0, 10, 9, 0, 0, 12]),
    'scatter_3d': _case(1888, [(F32, (4, 4, 4)), (I32, (2,)), (F32, (2, 4, 4))], lambda E, d, i, u: E.scatter(d, i, u),
                        [_Z64, [0, 2], _U32 * 2], np.array(_rows(_Z64, [(0, _U32), (2, _U32)])).reshape(4, 4, 4)),
    'scatter_dup_1d': _case(1917, [(F32, (8,)), (I32, (4,)), (F32, (4,))], lambda E, d, i, u: E.scatter(d, i, u),
                            [[0] * 8, [4, 3, 3, 7], [9, 10, 11, 12]], [0, 0, 0, 21, 9, 0, 0, 12]),
    'scatter_dup_3d': _case(1932, [(F32, (4, 4, 4)), (I32, (2,)), (F32, (2, 4, 4))], lambda E, d, i, u: E.scatter(d, i, u),
                            [_Z64, [2, 2], _U32 * 2], np.array(_rows(_Z64, [(2, [2 * v for v in _U32])])).reshape(4, 4, 4)),
    'scatter_1d_update_slice': _case(1962, [(F32, (8,)), (I32, (4,)), (F32, (4,))],
                                     lambda E, d, i, u: E.scatter(d, i, u, mode=E.SCATTER_UPDATE_SLICE),
                                     [[1] * 8, [4, 3, 1, 7], [9, 10, 11, 12]], [1, 11, 1, 10, 9, 1, 1, 12]),
    'scatter_3d_update_slice': _case(1976, [(F32, (4, 4, 4)), (I32, (2,)), (F32, (2, 4, 4))],
                                     lambda E, d, i, u: E.scatter(d, i, u, mode=E.SCATTER_UPDATE_SLICE),
                                     [_O64, [0, 2], _U32 * 2], np.array(_rows(_O64, [(0, _U32), (2, _U32)])).reshape(4, 4, 4)),
    'scatter_nd_update_slice': _case(2005, [(F32, (8,)), (I32, (4, 1)), (F32, (4,))],
                                     lambda E, d, i, u: E.scatter(d, i, u, mode=E.SCATTER_UPDATE_ND),
                                     [[1] * 8, [4, 3, 1, 7], [9, 10, 11, 12]], [1, 11, 1, 10, 9, 1, 1, 12]),
    'scatter_nd_update_slice2': _case(2020, [(F32, (4, 4, 4)), (I32, (2, 1)), (F32, (2, 4, 4))],
                                      lambda E, d, i, u: E.scatter(d, i, u, mode=E.SCATTER_UPDATE_ND),
                                      [_O64, [0, 2], _U32 * 2], np.array(_rows(_O64, [(0, _U32), (2, _U32)])).reshape(4, 4, 4)),
    'scatter_nd_update_slice3': _case(
        2050, [(F32, (1, 4, 4, 4)), (I32, (2, 3)), (F32, (2, 4))], lambda E, d, i, u: E.scatter(d, i, u, mode=E.SCATTER_UPDATE_ND),
        [_O64, [0, 0, 0, 0, 1, 2], [5] * 4 + [6] * 4],
        np.array([5] * 4 + [1] * 12 + [1] * 8 + [6] * 4 + [1] * 4 + [1] * 32).reshape(1, 4, 4, 4)),
    'scatter_elt': _case(2080, [(F32, (4, 4)), (I32, (2, 2)), (F32, (2, 2))],
                         lambda E, d, i, u: E.scatter(d, i, u, axis=1, mode=E.SCATTER_UPDATE_ELT),
                         [[1] * 16, [2, 0, 3, 1], [9] * 4], np.array([9, 1, 9, 1, 1, 9, 1, 9] + [1] * 8).reshape(4, 4)),
    'argsort_1d': _case(2400, [(F32, (20,))], lambda E, x: E.argsort(x, 0), [_SORT20], _ORDER20, out_dtype=np.int32),
    'argsort_1d_int': _case(2431, [(I32, (20,))], lambda E, x: E.argsort(x, 0),
                            [[81, 95, 27, 43, 55, 56, 57, 5, 39, 7, 14, 67, 20, 66, 64, 71, 68, 54, 87, 80]], _ORDER20,
                            out_dtype=np.int32),
    'argsort_1d_dup': _case(2462, [(F32, (20,))], lambda E, x: E.argsort(x, 0),
                            [[81.69, 81.69, 27.74, 43.69, 55.79, 56.79, 57.52, 7.11, 39.48, 5.9] + _SORT20[10:]],
                            [9, 7, 10, 12, 2, 8, 3, 17, 4, 5, 6, 14, 13, 11, 16, 15, 19, 0, 1, 18], out_dtype=np.int32),
    'argsort_2d_axis0': _case(2494, [(F32, (5, 4))], lambda E, x: E.argsort(x, 0), [_SORT20],
                              np.array([3, 2, 2, 1, 2, 4, 0, 0, 1, 1, 1, 2, 4, 3, 3, 3, 0, 0, 4, 4]).reshape(5, 4), out_dtype=np.int32),
    'argsort_2d_axis1': _case(2534, [(F32, (5, 4))], lambda E, x: E.argsort(x, 1), [_SORT20],
                              np.array([2, 3, 0, 1, 3, 0, 1, 2, 1, 2, 0, 3, 0, 2, 1, 3, 1, 0, 3, 2]).reshape(5, 4), out_dtype=np.int32),
}


def check_case(name, got):
    c = CASES[name]
    exp = c['expected']
    if exp.dtype == np.float16:
        got = got.astype(np.float16)   # the oracle carries 16-bit floats as rounded float32 values
    assert got.shape == exp.shape and got.dtype == exp.dtype, (name, got.shape, got.dtype, exp.shape, exp.dtype)
    if c['tol'] is None:
        np.testing.assert_array_equal(got, exp, err_msg=name)
    else:
        g, e = got.astype(np.float64), exp.astype(np.float64)
        bound = (np.abs(g) + np.abs(e)) * c['tol'] + 1e-6   # the expected values are printed with six digits
        assert (np.abs(g - e) <= bound).all(), (name, got, exp)


def build_case(name, E):
    c = CASES[name]
    ins, out = c['build'](E)
    return E.Program(name, ins, [out]), c['inputs']

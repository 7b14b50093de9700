"""argsort, gather and scatter: the oracle and the hip device against the reference tests' own answers
(tests/special_cases.py) and, on seeded inputs, against numpy closed forms and each other."""
import numpy as np
import pytest

import special_cases as SC
from oracle import tile_oracle as OE

NAMES = sorted(SC.CASES)


@pytest.mark.parametrize('name', NAMES)
def test_oracle_reproduces_reference_answers(name):
    prog, ins = SC.build_case(name, OE)
    SC.check_case(name, OE.run(prog, ins)[0])


def random_programs(E):
    """Larger seeded cases: (name, program, inputs, numpy expectation or None)."""
    r = np.random.default_rng(31)
    out = []
    x = r.integers(-5, 6, (7, 33, 5)).astype(np.float32)          # many ties
    X = E.Placeholder(E.DType.FLOAT32, [7, 33, 5])
    asc = np.argsort(x, axis=1, kind='stable').astype(np.int32)
    desc = np.flip(32 - np.argsort(np.flip(x, 1), axis=1, kind='stable'), 1).astype(np.int32)
    out.append(('argsort_ties', E.Program('p', [X], [E.argsort(x=X, axis=1), E.argsort(X, -2, E.SORT_DESC)]), [x], [asc, desc]))
    u = r.integers(0, 2 ** 63, (300,), dtype=np.uint64)
    u[7] = 2 ** 64 - 1
    U = E.Placeholder(E.DType.UINT64, [300])
    out.append(('argsort_u64', E.Program('p', [U], [E.argsort(U, 0, E.SORT_DESC)]), [u],
                [np.argsort(-u.astype(np.float64), kind='stable').astype(np.int32)]))
    t = r.standard_normal((4, 9, 6)).astype(np.float32)
    i = r.integers(0, 9, (5, 3)).astype(np.int32)
    T, I = E.Placeholder(E.DType.FLOAT32, [4, 9, 6]), E.Placeholder(E.DType.INT32, [5, 3])
    out.append(('gather_axis1', E.Program('p', [T, I], [E.gather(T, I, axis=1)]), [t, i], [np.take(t, i, axis=1)]))
    pos = r.uniform(-1.5, 9.5, (11,)).astype(np.float32)
    P = E.Placeholder(E.DType.FLOAT32, [11])
    lin = E.gather(T, P, axis=1, interpolation_mode=E.INTERP_LINEAR)
    cub = E.gather(T, P, axis=1, interpolation_mode=E.INTERP_CUBIC, out_of_bounds_mode=E.OOB_RETURN_ZERO)
    near = [E.gather(T, P, axis=1, interpolation_mode=E.INTERP_NEAREST, nearest_mode=m) for m in range(5)]
    out.append(('gather_interpolated', E.Program('p', [T, P], [lin, cub] + near), [t, pos], None))
    d = r.standard_normal((6, 5, 4)).astype(np.float32)
    si = r.integers(0, 5, (3, 2)).astype(np.int32)
    su = r.standard_normal((6, 3, 2, 4)).astype(np.float32)
    D, SI, SU = E.Placeholder(E.DType.FLOAT32, [6, 5, 4]), E.Placeholder(E.DType.INT32, [3, 2]), E.Placeholder(E.DType.FLOAT32, [6, 3, 2, 4])
    di = r.integers(-100, 100, (6, 5, 4)).astype(np.int32)
    ui = r.integers(-100, 100, (3, 2, 4)).astype(np.int32)
    ii = r.integers(0, 6, (3, 2)).astype(np.int32)
    DI, II, UI = E.Placeholder(E.DType.INT32, [6, 5, 4]), E.Placeholder(E.DType.INT32, [3, 2]), E.Placeholder(E.DType.INT32, [3, 2, 4])
    ref = di.copy()
    np.add.at(ref, (ii[:, :, None], np.arange(2)[None, :, None], np.arange(4)[None, None, :]), ui)
    out.append(('scatter_add_int_dups', E.Program('p', [DI, II, UI], [E.scatter(DI, II, UI)]), [di, ii, ui], [ref]))
    # scatter-add on the narrow and wide element types (compare-and-swap paths on the device); small integers, so
    # that every partial sum is exact whatever order the duplicates arrive in
    for dt_name, npdt in (('BFLOAT16', np.float32), ('INT8', np.int8), ('FLOAT64', np.float64), ('INT64', np.int64), ('FLOAT16', np.float16)):
        base = r.integers(-3, 4, (5, 7)).astype(npdt)
        upd = r.integers(-2, 3, (9, 7)).astype(npdt)
        idx = r.integers(0, 5, (9,)).astype(np.int32)
        Dd, Ii, Uu = (E.Placeholder(getattr(E.DType, dt_name), [5, 7]), E.Placeholder(E.DType.INT32, [9]),
                      E.Placeholder(getattr(E.DType, dt_name), [9, 7]))
        want = base.astype(np.float64).copy()
        np.add.at(want, idx, upd.astype(np.float64))
        out.append(('scatter_add_' + dt_name.lower(), E.Program('p', [Dd, Ii, Uu], [E.scatter(Dd, Ii, Uu)]), [base, idx, upd],
                    [want.astype(npdt)]))
    # a line longer than the device stages in LDS
    long_line = r.integers(0, 50, (2, 9000)).astype(np.int32)
    LL = E.Placeholder(E.DType.INT32, [2, 9000])
    out.append(('argsort_long_line', E.Program('p', [LL], [E.argsort(LL, 1)]), [long_line],
                [np.argsort(long_line, axis=1, kind='stable').astype(np.int32)]))
    return out, (D, SI, SU, d, si, su)


def test_oracle_matches_numpy_on_seeded_cases():
    progs, _ = random_programs(OE)
    for name, prog, ins, refs in progs:
        outs = OE.run(prog, ins)
        if refs is not None:
            for o, r in zip(outs, refs):
                np.testing.assert_array_equal(o, r, err_msg=name)


def test_oracle_linear_gather_is_piecewise_linear_interpolation():
    """Inside the range the LINEAR mode equals numpy's interp; outside it holds the edge value (or zero)."""
    t = np.array([0.5, -2.0, 4.0, 1.0, 3.5], np.float32)
    pos = np.linspace(-1, 5, 25).astype(np.float32)
    T, P = OE.Placeholder(OE.DType.FLOAT32, [5]), OE.Placeholder(OE.DType.FLOAT32, [25])
    edge, zero = OE.run(OE.Program('p', [T, P], [OE.gather(T, P, interpolation_mode=OE.INTERP_LINEAR),
                                                 OE.gather(T, P, interpolation_mode=OE.INTERP_LINEAR,
                                                           out_of_bounds_mode=OE.OOB_RETURN_ZERO)]), [t, pos])
    want = np.interp(pos, np.arange(5), t)
    np.testing.assert_allclose(edge, want, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(zero, np.where((pos < 0) | (pos > 4), 0, want), rtol=1e-6, atol=1e-6)


def test_oracle_cubic_gather_reproduces_cubics_exactly_at_interior_points():
    """Keys' cubic convolution with a = -0.5 reproduces any quadratic between interior samples."""
    k = np.arange(8, dtype=np.float64)
    t = (0.25 * k * k - k + 2).astype(np.float64)
    pos = np.linspace(1, 6, 21)
    T, P = OE.Placeholder(OE.DType.FLOAT64, [8]), OE.Placeholder(OE.DType.FLOAT64, [21])
    got, = OE.run(OE.Program('p', [T, P], [OE.gather(T, P, interpolation_mode=OE.INTERP_CUBIC, cube_coeff=-0.5)]), [t, pos])
    np.testing.assert_allclose(got, 0.25 * pos * pos - pos + 2, rtol=1e-12, atol=1e-12)


@pytest.mark.gpu
@pytest.mark.parametrize('name', NAMES)
def test_hip_reproduces_reference_answers(name):
    from plaidml_amd import edsl as E
    print('special case', name, flush=True)
    prog, ins = SC.build_case(name, E)
    got = E.run(prog, ins, target='hip')[0]
    SC.check_case(name, got)
    oprog, oins = SC.build_case(name, OE)
    ref = OE.run(oprog, oins)[0]
    if SC.CASES[name]['tol'] is None:
        np.testing.assert_array_equal(got, ref)
    else:
        np.testing.assert_allclose(got.astype(np.float64), ref.astype(np.float64), rtol=2e-3 if got.dtype == np.float16 else 1e-6,
                                   atol=1e-6)


@pytest.mark.gpu
def test_hip_matches_oracle_on_seeded_cases():
    from plaidml_amd import edsl as E
    progs, _ = random_programs(E)
    oprogs, _ = random_programs(OE)
    for (name, prog, ins, refs), (_, oprog, oins, _) in zip(progs, oprogs):
        print('seeded special case', name, flush=True)
        outs = E.run(prog, ins, target='hip')
        want = OE.run(oprog, oins)
        for k, (o, w) in enumerate(zip(outs, want)):
            if name == 'gather_interpolated':
                np.testing.assert_allclose(o, w, rtol=1e-6, atol=1e-6, err_msg='%s output %d' % (name, k))
            else:
                np.testing.assert_array_equal(o, w, err_msg='%s output %d' % (name, k))


@pytest.mark.gpu
def test_hip_index_outside_the_tensor_reads_zero_and_drops_updates():
    """Undefined in the reference; this device never touches memory outside the tensors."""
    from plaidml_amd import edsl as E
    T, I = E.Placeholder(E.DType.FLOAT32, [4]), E.Placeholder(E.DType.INT32, [3])
    U = E.Placeholder(E.DType.FLOAT32, [3])
    g, s = E.run(E.Program('p', [T, I, U], [E.gather(T, I), E.scatter(T, I, U)]),
                 [np.arange(1, 5, dtype=np.float32), np.array([2, 9, -1], np.int32), np.array([10, 20, 30], np.float32)], target='hip')
    np.testing.assert_array_equal(g, [3, 0, 0])
    np.testing.assert_array_equal(s, [1, 2, 13, 4])


# CppEdsl.Prng, plaidml/edsl/tests/edsl_test.cc:1138-1160: state {5, 6, 7}, six values, the state after them
PRNG_VALUES = np.array([9.31323e-10, 3.8147e-06, 0.0156251, 0.000244171, 0.000125885, 0.515625], np.float32).reshape(2, 3)
PRNG_STATE = np.array([1052804, 0, 0], np.uint32).reshape(1, 3)


def _prng_program(E, dims):
    S = E.Placeholder(E.DType.UINT32, [1, 3])
    vals, new_state = E.prng(S, dims)
    return E.Program('prng', [S], [vals, new_state])


def test_oracle_prng_reproduces_reference_answers():
    vals, st = OE.run(_prng_program(OE, [2, 3]), [np.array([[5, 6, 7]], np.uint32)])
    np.testing.assert_allclose(vals, PRNG_VALUES, rtol=1e-5)
    np.testing.assert_array_equal(st, PRNG_STATE)


def test_oracle_prng_streams_compose():
    """Drawing n values and then m from the returned state equals drawing n + m at once."""
    s = np.array([[123456789, 362436069, 521288629]], np.uint32)
    a, sa = OE.run(_prng_program(OE, [100]), [s])
    b, sb = OE.run(_prng_program(OE, [57]), [sa])
    c, sc = OE.run(_prng_program(OE, [157]), [s])
    np.testing.assert_array_equal(np.concatenate([a, b]), c)
    np.testing.assert_array_equal(sb, sc)
    assert 0.0 <= c.min() and c.max() <= 1.0   # a quotient just below 1 rounds to 1.0f, as in the reference
    assert abs(c.mean() - 0.5) < 0.1


@pytest.mark.gpu
def test_hip_prng_matches_reference_answers_and_oracle():
    from plaidml_amd import edsl as E
    vals, st = E.run(_prng_program(E, [2, 3]), [np.array([[5, 6, 7]], np.uint32)], target='hip')
    np.testing.assert_allclose(vals, PRNG_VALUES, rtol=1e-5)
    np.testing.assert_array_equal(st, PRNG_STATE)
    # a count that spans many threads and is not a multiple of a thread's run: bit-exact against the serial oracle
    s = np.array([[123456789, 362436069, 521288629]], np.uint32)
    got, gst = E.run(_prng_program(E, [7, 1001]), [s], target='hip')
    want, wst = OE.run(_prng_program(OE, [7, 1001]), [s])
    np.testing.assert_array_equal(got, want)
    np.testing.assert_array_equal(gst, wst)

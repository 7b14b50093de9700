"""Pins the CPU oracle against the reference's own known-answer vectors.

Each expected vector below is data held by a reference test (file:line given at
each case); none of them is computed by the oracle's own formulas.
"""
import numpy as np
import pytest

from oracle import tile_oracle as E
from oracle import tile_oplib as op

D = E.DType


def gemm(A, B, C):
    # plaidml/edsl/examples/gemm.cc:16-22
    I, J, K = E.TensorDims(3)
    i, j, k = E.TensorIndexes(3)
    A.bind_dims(I, K)
    B.bind_dims(K, J)
    return E.Contraction().outShape(I, J).outAccess(i, j).sum(A[i, k] * B[k, j]).build() + C


@pytest.mark.parametrize('dt,npdt,a,b,o', [
    # plaidml/edsl/examples/gemm.cc:27-77
    (D.INT64, np.int64, [1, 1, 1, 1, 1, 2, 3, 3, 3], [10, 11, 12, 13, 14, 15, 16, 17, 18],
     [40, 43, 46, 56, 60, 64, 118, 127, 136]),
    (D.UINT64, np.uint64, [1, 1, 1, 1, 1, 2, 3, 3, 3], [10, 11, 12, 13, 14, 15, 16, 17, 18],
     [40, 43, 46, 56, 60, 64, 118, 127, 136]),
    (D.INT32, np.int32, [1, 1, 1, 1, 1, 2, 3, 3, 3], [10, 11, 12, 13, 14, 15, 16, 17, 18],
     [40, 43, 46, 56, 60, 64, 118, 127, 136]),
    (D.INT8, np.int8, [1, 1, 1, 1, 1, 2, 3, 3, 3], [1, 2, 3, 3, 4, 5, 3, 3, 3],
     [8, 10, 12, 11, 13, 15, 22, 28, 34]),
])
def test_gemm_int_exact(dt, npdt, a, b, o):
    A, B, C = (E.Placeholder(dt, [3, 3]) for _ in range(3))
    prog = E.Program('gemm', [A, B, C], [gemm(A, B, C)])
    out, = E.run(prog, [np.array(a, npdt), np.array(b, npdt), np.ones(9, npdt)])
    assert out.dtype == npdt
    np.testing.assert_array_equal(out.reshape(-1), np.array(o, npdt))


def test_gemm_float32():
    # plaidml/edsl/examples/gemm.cc:79-90
    A, B, C = (E.Placeholder(D.FLOAT32, [3, 3]) for _ in range(3))
    prog = E.Program('gemm', [A, B, C], [gemm(A, B, C)])
    out, = E.run(prog, [np.array([0.5, 0.2, 4, 1, 1, 2, 3, 3, 0.3], np.float32),
                        np.array([1, 2, 3, 3, 4, 0.5, 3, 3, 3], np.float32), np.ones(9, np.float32)])
    exp = np.array([14.1, 14.8, 14.6, 11, 13, 10.5, 13.9, 19.9, 12.4], np.float32)
    np.testing.assert_allclose(out.reshape(-1), exp, rtol=1e-6)


def test_int8_gemm_wraps_in_int8():
    # the accumulator is not widened (pmlc/ast/eval.cc:22-44; ConvI8 result is si8,
    # plaidml/edsl/tests/edsl_test.cc:1195-1208): 100*2 + 100*2 = 400 -> 400 - 512 = -112
    A, B, C = (E.Placeholder(D.INT8, [1, 2]), E.Placeholder(D.INT8, [2, 1]), E.Placeholder(D.INT8, [1, 1]))
    prog = E.Program('gemm', [A, B, C], [gemm(A, B, C)])
    out, = E.run(prog, [np.array([100, 100], np.int8), np.array([2, 2], np.int8), np.zeros(1, np.int8)])
    assert out.dtype == np.int8 and int(out[0, 0]) == -112


def test_funky_sum():
    # plaidml/edsl/tests/edsl_test.cc:2709-2719 / edsl_test.py:408-419 (test_defract)
    I = E.Placeholder(D.FLOAT32, [3])
    K = E.Placeholder(D.FLOAT32, [3])
    i, j = E.TensorIndexes(2)
    O = E.Contraction().outShape(5).outAccess(i).sum(I[(i - j + 1) // 2] * K[j]).build()
    out, = E.run(E.Program('funky_sum', [I, K], [O]), [np.array([1, 2, 3], np.float32)] * 2)
    np.testing.assert_array_equal(out, np.array([2, 5, 4, 9, 6], np.float32))


def test_defract_short():
    # plaidml/edsl/tests/edsl_test.py:421-431
    I = E.Placeholder(D.FLOAT32, [3])
    i, j = E.TensorIndexes(2)
    O = E.Contraction().outShape(6).outAccess(i).sum(I[(i - 1) // 2]).build()
    out, = E.run(E.Program('defract_short_test', [I], [O]), [np.array([1, 2, 3], np.float32)])
    np.testing.assert_array_equal(out, np.array([0, 1, 0, 2, 0, 3], np.float32))


def test_defract_long():
    # plaidml/edsl/tests/edsl_test.py:433-460
    shape = [1, 3, 3, 1]
    I = E.Placeholder(D.FLOAT32, shape)
    K = E.Placeholder(D.FLOAT32, shape)
    n, x0, x1, c0, c1, co, ci, k0, k1 = E.TensorIndexes(9)
    O = E.Contraction().outShape(1, 5, 5, 1).outAccess(n, x0, x1, co).sum(
        I[n, (x0 + k0 - 1) // 2, (x1 + k1 - 1) // 2, ci] * K[2 - k0, 2 - k1, co, ci]).build()
    out, = E.run(E.Program('defract_long', [I, K], [O]), [
        np.array([[[[1], [3], [-1]], [[0], [2], [4]], [[1], [-1], [-2]]]], np.float32),
        np.array([[[[2], [3], [4]], [[6], [-3], [-1]], [[-1], [-2], [1]]]], np.float32)])
    exp = np.array([[[[0], [0], [0], [0], [0]], [[0], [4], [12], [6], [24]], [[0], [0], [0], [0], [0]],
                     [[6], [-3], [-6], [-3], [-12]], [[0], [0], [0], [0], [0]]]], np.float32)
    np.testing.assert_array_equal(out, exp)


def test_max_rows():
    # plaidml/edsl/tests/edsl_test.cc:576-590
    A = E.Placeholder(D.FLOAT32, [3, 3])
    i, j = E.TensorIndexes(2)
    R = E.Contraction().outShape(3).outAccess(i).max(A[i, j]).build()
    out, = E.run(E.Program('max', [A], [R]), [np.array([-5, -6, -7, 4, 5, 6, 7, 8, 9], np.float32)])
    np.testing.assert_array_equal(out, np.array([-5, 6, 9], np.float32))


def test_quantize_truncates():
    # plaidml/edsl/examples/quantize.cc:16-32
    A = E.Placeholder(D.FLOAT32, [3])
    O = E.cast(A * 256.0, D.INT8) + 0
    out, = E.run(E.Program('quantize', [A], [O]), [np.array([0.1, 0.4, 0.3], np.float32)])
    assert out.dtype == np.int8
    np.testing.assert_array_equal(out, np.array([25, 102, 76], np.int8))


def test_higher_precision_constants():
    # plaidml/edsl/tests/edsl_test.cc:140-156
    A = E.Placeholder(D.FLOAT32, [3, 3])
    C = A + E.cast(E.Constant(1), D.UINT64) + E.cast(E.Constant(2.0), D.FLOAT64)
    out, = E.run(E.Program('hpc', [A], [C]), [np.arange(1, 10, dtype=np.float32)])
    assert out.dtype == np.float64
    np.testing.assert_array_equal(out.reshape(-1), np.arange(4, 13, dtype=np.float64))


def test_cast_u64_u32():
    # plaidml/edsl/tests/edsl_test.cc:158-182
    A = E.Placeholder(D.UINT64, [3, 3])
    vals = [1, 2, 3, 4, 5, 6 + (1 << 12), 7 + (1 << 24), 8 + (1 << 31), (1 << 32) - 1]
    out, = E.run(E.Program('cast', [A], [E.cast(A, D.UINT32)]), [np.array(vals, np.uint64)])
    assert out.dtype == np.uint32
    np.testing.assert_array_equal(out.reshape(-1), np.array(vals, np.uint32))


def test_broadcast_cmp():
    # plaidml/edsl/tests/edsl_test.cc:319-333
    A = E.Placeholder(D.UINT64, [3, 4])
    B = E.Placeholder(D.UINT64, [3, 1])
    C = E.cast(A >= B, D.UINT64)
    out, = E.run(E.Program('broadcast_cmp', [A, B], [C]),
                 [np.arange(12, dtype=np.uint64), np.array([0, 6, 12], np.uint64)])
    np.testing.assert_array_equal(out.reshape(-1), np.array([1, 1, 1, 1, 0, 0, 1, 1, 0, 0, 0, 0], np.uint64))


def test_add_u64():
    # plaidml/edsl/tests/edsl_test.cc:335-374
    a = [1, 2, 3, 4, 5, 6 + (1 << 12), 7 + (1 << 24), 8 + (1 << 32), 9 + (1 << 40)]
    b = [1, 2 + (1 << 12), 3, 4 + (1 << 24), 5, 6 + (1 << 32), 7, 8 + (1 << 40), 9]
    c = [2, 4 + (1 << 12), 6, 8 + (1 << 24), 10, 12 + (1 << 12) + (1 << 32), 14 + (1 << 24),
         16 + (1 << 32) + (1 << 40), 18 + (1 << 40)]
    A = E.Placeholder(D.UINT64, [3, 3])
    B = E.Placeholder(D.UINT64, [3, 3])
    out, = E.run(E.Program('add', [A, B], [A + B]), [np.array(a, np.uint64), np.array(b, np.uint64)])
    np.testing.assert_array_equal(out.reshape(-1), np.array(c, np.uint64))


def test_mixed_add():
    # plaidml/edsl/tests/edsl_test.cc:396-408: si32 constants + ui32 input -> ui32
    I = E.Placeholder(D.UINT32, [4])
    A = E.Constant(np.array([4, 3, 2, 1], np.int32))
    B = E.Constant(np.array([1, 2, 3, 4], np.int32))
    O = (A + B) + I
    out, = E.run(E.Program('mixed_add', [I], [O]), [np.array([1, 2, 2, 1], np.uint32)])
    assert out.dtype == np.uint32
    np.testing.assert_array_equal(out, np.array([6, 7, 7, 6], np.uint32))


def test_round_half_away():
    # plaidml/edsl/tests/edsl_test.cc:1820-1835
    S = E.Placeholder(D.FLOAT32, [3, 3])
    out, = E.run(E.Program('round', [S], [E.round(S)]),
                 [np.array([1.1, 9.21, 3.0, -0.4, -7.0, 0.6, 1.0, 0.0, -6.6], np.float32)])
    np.testing.assert_array_equal(out.reshape(-1), np.array([1, 9, 3, -0, -7, 1, 1, 0, -7], np.float32))


# --- closed-form goldens of pmlc/target/x86/tests/xsmm_call.mlir -------------------------------


def test_xsmm_call_dot_rows():
    # fill_2d (:96-116): A[x,y] = x+y-5 ; B[x,y] = x+y+(8x+y)-5 ; CHECK rows :163-170
    x, y = np.meshgrid(np.arange(8), np.arange(8), indexing='ij')
    Av = (x + y - 5).astype(np.float32)
    Bv = (x + y + (x * 8 + y) - 5).astype(np.float32)
    A = E.Placeholder(D.FLOAT32, [8, 8])
    B = E.Placeholder(D.FLOAT32, [8, 8])
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(8, 8).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    out, = E.run(E.Program('dot', [A, B], [C]), [Av, Bv])
    rows = {0: [60, 36, 12, -12, -36, -60, -84, -108], 1: [272, 264, 256, 248, 240, 232, 224, 216],
            4: [908, 948, 988, 1028, 1068, 1108, 1148, 1188], 7: [1544, 1632, 1720, 1808, 1896, 1984, 2072, 2160]}
    for r, exp in rows.items():
        np.testing.assert_array_equal(out[r], np.array(exp, np.float32))


def test_xsmm_call_conv_rows():
    # fill_4d (:118-142): I[x,y,z,w] = x+y+z+w-5 ; K = x+y+z+w + (x*Y + y*W + z*W + w) - 5 ; CHECK :229-258
    def fill(shape, alt):
        X, Y, Z, W = shape
        x, y, z, w = np.meshgrid(*[np.arange(s) for s in shape], indexing='ij')
        i = x * Y + y * W + z * W + w
        return (x + y + z + w + (i if alt else 0) - 5).astype(np.float32)

    Iv, Kv = fill((1, 6, 5, 7), False), fill((1, 1, 7, 11), True)
    I = E.Placeholder(D.FLOAT32, [1, 6, 5, 7])
    K = E.Placeholder(D.FLOAT32, [1, 1, 7, 11])
    O = op.convolution(I, K, autopad=op.VALID)
    out, = E.run(E.Program('conv2', [I, K], [O]), [Iv, Kv])
    assert out.shape == (1, 6, 5, 11)
    np.testing.assert_array_equal(out[0, 0, 0], np.array([-98, -126, -154, -182, -210, -238, -266, -294, -322, -350, -378], np.float32))
    np.testing.assert_array_equal(out[0, 0, 1], np.array([119, 105, 91, 77, 63, 49, 35, 21, 7, -7, -21], np.float32))
    np.testing.assert_array_equal(out[0, 0, 2], np.full(11, 336, np.float32))
    np.testing.assert_array_equal(out[0, 5, 4], np.array([1855, 1953, 2051, 2149, 2247, 2345, 2443, 2541, 2639, 2737, 2835], np.float32))
    np.testing.assert_array_equal(out[0, 3, 2], np.array([987, 1029, 1071, 1113, 1155, 1197, 1239, 1281, 1323, 1365, 1407], np.float32))


# --- what the mathematics fixes: textbook reductions and brute force ------------------------------


def test_bounds_box_of_same_conv():
    # SAME 3x3 conv: k in [0,2], x in [0,H-1]; the residual constraint 0 <= x+k-1 <= H-1 drops the edge taps
    I = E.Placeholder(D.FLOAT32, [1, 5, 5, 2])
    F = E.Placeholder(D.FLOAT32, [3, 3, 2, 3])
    O = op.convolution(I, F)
    a = O.attrs
    rng = np.random.default_rng(0)
    Iv = rng.standard_normal((1, 5, 5, 2)).astype(np.float32)
    Fv = rng.standard_normal((3, 3, 2, 3)).astype(np.float32)
    out, box, n = E.contract(a['agg'], a['combo'], O.dt, O.shape, a['sink'], [(Iv, D.FLOAT32), (Fv, D.FLOAT32)],
                             a['accs'], a['cons'], None, return_box=True)
    assert sorted(box.values()) == sorted([(0, 0), (0, 4), (0, 4), (0, 2), (0, 2), (0, 2), (0, 1)])
    # valid taps per spatial dim = 3*5 - 2
    assert n == (3 * 5 - 2) ** 2 * 2 * 3


@pytest.mark.parametrize('stride,autopad,k', [(1, op.SAME_UPPER, 3), (2, op.SAME_UPPER, 3), (2, op.VALID, 3),
                                               (2, op.SAME_UPPER, 7), (1, op.SAME_LOWER, 2), (2, op.SAME_UPPER, 1)])
def test_conv_matches_torch(stride, autopad, k):
    import torch
    import torch.nn.functional as F_
    rng = np.random.default_rng(1)
    H = 9
    Iv = rng.standard_normal((2, H, H, 3)).astype(np.float32)
    Fv = rng.standard_normal((k, k, 3, 4)).astype(np.float32)
    I = E.Placeholder(D.FLOAT32, Iv.shape)
    F = E.Placeholder(D.FLOAT32, Fv.shape)
    O = op.convolution(I, F, strides=[stride, stride], autopad=autopad)
    out, = E.run(E.Program('conv', [I, F], [O]), [Iv, Fv])
    pad, osz = op.compute_padding_and_output_size(H, k, stride, autopad)
    total = max(0, (osz - 1) * stride + k - H) if autopad != op.VALID else 0
    x = torch.from_numpy(Iv).permute(0, 3, 1, 2).double()
    x = F_.pad(x, (pad, total - pad, pad, total - pad))
    ref = F_.conv2d(x, torch.from_numpy(Fv).permute(3, 2, 0, 1).double(), stride=stride).permute(0, 2, 3, 1).numpy()
    assert out.shape == ref.shape
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5)


def test_depthwise_matches_torch():
    import torch
    import torch.nn.functional as F_
    rng = np.random.default_rng(2)
    C = 5
    Iv = rng.standard_normal((2, 7, 7, C)).astype(np.float32)
    Fv = rng.standard_normal((3, 3, C, 1)).astype(np.float32)
    I = E.Placeholder(D.FLOAT32, Iv.shape)
    F = E.Placeholder(D.FLOAT32, Fv.shape)
    O = op.convolution(I, F, depthwise=True)
    out, = E.run(E.Program('dw', [I, F], [O]), [Iv, Fv])
    ref = F_.conv2d(torch.from_numpy(Iv).permute(0, 3, 1, 2).double(),
                    torch.from_numpy(Fv).permute(2, 3, 0, 1).double(), padding=1, groups=C).permute(0, 2, 3, 1).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-4, atol=1e-5)


def test_maxpool_values_match_torch_and_argmax_ties():
    import torch
    import torch.nn.functional as F_
    rng = np.random.default_rng(3)
    Iv = rng.integers(-3, 4, size=(2, 7, 7, 3)).astype(np.float32)  # many ties
    I = E.Placeholder(D.FLOAT32, Iv.shape)
    M = op.pool(I, 'max', [3, 3], [2, 2], autopad=op.SAME_UPPER)
    n, x0, x1, c, k0, k1 = E.TensorIndexes(6)
    IX = E.index([3, 3], 0) * 3 + E.index([3, 3], 1)
    AM = E.Contraction().outShape(M.shape).outAccess(n, x0, x1, c).max(
        E.cond(I[n, 2 * x0 + k0 - 1, 2 * x1 + k1 - 1, c], M[n, x0, x1, c], IX[k0, k1])).build()
    m, am = E.run(E.Program('pool', [I], [M, AM]), [Iv])
    ref = F_.max_pool2d(torch.from_numpy(Iv).permute(0, 3, 1, 2), 3, 2, padding=1).permute(0, 2, 3, 1).numpy()
    np.testing.assert_array_equal(m, ref)
    assert am.dtype == np.int32
    # brute force: the largest window index whose tap is in bounds and equals the max
    exp = np.zeros(m.shape, np.int32)
    for idx in np.ndindex(*m.shape):
        b, y, x, ch = idx
        best = 0
        for a in range(3):
            for bb in range(3):
                yy, xx = 2 * y + a - 1, 2 * x + bb - 1
                if 0 <= yy < 7 and 0 <= xx < 7 and Iv[b, yy, xx, ch] == m[idx]:
                    best = max(best, a * 3 + bb)
        exp[idx] = best
    np.testing.assert_array_equal(am, exp)


def test_max_ignores_nan_and_int_identity_quirk():
    A = E.Placeholder(D.FLOAT32, [1, 3])
    i, j = E.TensorIndexes(2)
    R = E.Contraction().outShape(1).outAccess(i).max(A[i, j]).build()
    out, = E.run(E.Program('max', [A], [R]), [np.array([[1.0, np.nan, 0.5]], np.float32)])
    assert out[0] == 1.0
    # signed 32-bit max starts from int64 min truncated to 32 bits = 0
    B = E.Placeholder(D.INT32, [1, 2])
    R2 = E.Contraction().outShape(1).outAccess(i).max(B[i, j]).build()
    out2, = E.run(E.Program('max', [B], [R2]), [np.array([[-4, -2]], np.int32)])
    assert int(out2[0]) == 0


def test_softmax_mean_argmax_closed_forms():
    rng = np.random.default_rng(4)
    Xv = rng.standard_normal((4, 10)).astype(np.float32)
    X = E.Placeholder(D.FLOAT32, Xv.shape)
    s, m, am = E.run(E.Program('t', [X], [op.softmax(X, 1), op.mean(X, [1]), op.argmax(X, 1)]), [Xv])
    e = np.exp(Xv - Xv.max(1, keepdims=True))
    np.testing.assert_allclose(s, e / e.sum(1, keepdims=True), rtol=1e-6)
    np.testing.assert_allclose(m, Xv.mean(1), rtol=1e-5, atol=1e-6)
    assert am.dtype == np.uint32
    np.testing.assert_array_equal(am, Xv.argmax(1).astype(np.uint32))


def test_bf16_rounding_is_nearest_even():
    a = np.array([1.0, 1.00390625, 1.01171875, -2.5, 3.4e38], np.float32)
    # 1 + 2^-8 is a tie between 1.0 and 1+2^-7 -> even mantissa (1.0); 1+3*2^-8 ties up to 1+2^-6
    r = E.round_bf16(a)
    assert r[0] == 1.0 and r[1] == 1.0 and r[2] == np.float32(1.015625) and r[3] == -2.5
    assert np.isinf(r[4])
    np.testing.assert_array_equal(E.bf16_from_bits(E.bf16_bits(r[:4])), r[:4])


@pytest.mark.parametrize('dtype_name', ['INT64', 'UINT64', 'INT32', 'INT8', 'FLOAT32'])
def test_gemv_known_answers(dtype_name):
    """plaidml/edsl/examples/gemv.cc:39-139: A x + y for five element types, and (5 A) x + 4 y = 19 19 19."""
    import programs
    from oracle import tile_oplib as Oop
    prog, vals, _ = programs.gemv(E, Oop, dtype_name)
    o, o2, p = E.run(prog, vals)
    want = np.array(programs.GEMV_ANSWERS[dtype_name][1], o.dtype)
    np.testing.assert_array_equal(o, want)
    if dtype_name == 'INT64':
        np.testing.assert_array_equal(o2, [19, 19, 19])
    np.testing.assert_array_equal(p, [1])


def test_bf16_contractions_round_once_after_the_last_tap():
    """What the declared bf16 semantics fix (fp32 accumulation, one rounding to nearest even at the end, the
    initial value inside the accumulator), on sums that fp32 holds exactly and bf16 does not: rounding after
    every tap, after partial sums, or before the initial value goes in gives 256 / 258 / 128 instead."""
    import programs
    from oracle import tile_oplib as Oop
    prog, vals, _ = programs.bf16_rounding_placement(E, Oop)
    for got, want in zip(E.run(prog, vals), programs.BF16_ROUNDING_ANSWERS):
        np.testing.assert_array_equal(got, want)


def test_f16_contraction_rounds_once():
    """The same for fp16 (11 significant bits): 2048 + 1 + 1 + 1 = 2051 -> 2052 (per tap: 2048)."""
    A = E.Placeholder(D.FLOAT16, [1, 4])
    B = E.Placeholder(D.FLOAT16, [4, 1])
    i, j, k = E.TensorIndexes(3)
    O = E.Contraction().outShape(1, 1).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    out, = E.run(E.Program('f16', [A, B], [O]), [np.array([[2048, 1, 1, 1]], np.float16), np.ones((4, 1), np.float16)])
    assert float(out[0, 0]) == 2052.0


def test_eq_combination_closed_forms():
    """`eq` (edsl.h:421; i1 result: eval.cc:25; tile_to_linalg.cc:1257-1262): any / all / parity of the match
    table by numpy, NaN never equal, uncovered elements hold min's identity (true)."""
    import programs
    from oracle import tile_oplib as Oop
    prog, vals, _ = programs.eq_combination(E, Oop)
    outs = E.run(prog, vals)
    want = programs.eq_combination_answers(*vals)
    assert len(outs) == len(want)
    for k, (g, w) in enumerate(zip(outs, want)):
        assert g.dtype == np.bool_ and g.shape == w.shape, k
        np.testing.assert_array_equal(g, w, err_msg=str(k))
    assert outs[0].any() and not outs[1].all() and outs[2].any() and not outs[2].all()  # the case is telling


def test_output_accesses_that_are_sums_of_indices():
    """The oracle on output coordinates that are sums of indices, against closed forms: the flattening contraction of
    compute-bounds.mlir:34-45 is a reshape; a transposed convolution written from the input's side equals explicit
    loops over the input pixels; a mirrored, strided coordinate equals a direct double loop."""
    import programs
    from oracle import tile_oplib as Oop
    prog, vals, _ = programs.flatten_by_contraction(E, Oop)
    np.testing.assert_array_equal(E.run(prog, vals)[0], vals[0].reshape(100))
    prog, vals, _ = programs.scatter_form_transposed_conv(E, Oop)
    want = programs.scatter_form_transposed_conv_answer(*vals)
    got, = E.run(prog, vals)
    np.testing.assert_array_equal(got, want.astype(np.float32))
    assert np.count_nonzero(want[:, -1]) and np.count_nonzero(want[:, :, -1])  # the last row / column is reached
    prog, vals, _ = programs.mirrored_sum_of_indices(E, Oop)
    A, B = vals
    want = np.zeros((14, 5), np.int64)
    for i in range(6):
        for j in range(4):
            want[7 - i + 2 * j] += A[i].astype(np.int64) * B[j]
    np.testing.assert_array_equal(E.run(prog, vals)[0], want.astype(np.int32))

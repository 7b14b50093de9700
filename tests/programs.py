"""Tile programs written once and built twice: with the CPU oracle's EDSL (oracle.tile_oracle /
oracle.tile_oplib) and with the product's EDSL (plaidml_amd.edsl / plaidml_amd.op, i.e. the plaidml_*
C ABI).  Each builder takes the two modules and returns (program, input arrays, tolerance class).

Programs restate the reference's own tests where one exists (file:line in each docstring) and the
five workload configurations of this build at reduced sizes.
"""
import numpy as np

EXACT, FP32, BF16 = 'exact', 'fp32', 'bf16'


def _rng(seed):
    return np.random.default_rng(seed)


def _bf16(a):
    from oracle.tile_oracle import round_bf16
    return round_bf16(np.asarray(a, np.float32))


def dot_f32(E, op, M=8, N=32, K=16, seed=2):
    """CppEdsl.Dot, plaidml/edsl/tests/edsl_test.cc:448-486 (8x16 . 16x32, normal(0,1) inputs)."""
    A = E.Placeholder(E.DType.FLOAT32, [M, K])
    B = E.Placeholder(E.DType.FLOAT32, [K, N])
    I, J, Kd = E.TensorDims(3)
    i, j, k = E.TensorIndexes(3)
    A.bind_dims(I, Kd)
    B.bind_dims(Kd, J)
    C = E.Contraction().outShape(I, J).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    r = _rng(seed)
    return E.Program('dot', [A, B], [C]), [r.standard_normal((M, K)).astype(np.float32),
                                           r.standard_normal((K, N)).astype(np.float32)], FP32


def gemm_int(E, op, dtype_name='INT32'):
    """ExampleCppEdsl.GEMM_*, plaidml/edsl/examples/gemm.cc:16-77: contraction + C, integer types."""
    dt = getattr(E.DType, dtype_name)
    npdt = {'INT64': np.int64, 'UINT64': np.uint64, 'INT32': np.int32, 'INT8': np.int8}[dtype_name]
    A, B, C = (E.Placeholder(dt, [3, 3]) for _ in range(3))
    i, j, k = E.TensorIndexes(3)
    O = E.Contraction().outShape(3, 3).outAccess(i, j).sum(A[i, k] * B[k, j]).build() + C
    a = np.array([1, 1, 1, 1, 1, 2, 3, 3, 3], npdt).reshape(3, 3)
    b = (np.array([1, 2, 3, 3, 4, 5, 3, 3, 3], npdt) if dtype_name == 'INT8'
         else np.array([10, 11, 12, 13, 14, 15, 16, 17, 18], npdt)).reshape(3, 3)
    return E.Program('gemm', [A, B, C], [O]), [a, b, np.ones((3, 3), npdt)], EXACT


GEMV_ANSWERS = {  # dtype -> (A, answer); x = y = ones: plaidml/edsl/examples/gemv.cc:56-139
    'INT64': ([1] * 9, [4, 4, 4]), 'UINT64': ([1] * 9, [4, 4, 4]), 'INT32': ([1] * 9, [4, 4, 4]),
    'INT8': ([1] * 9, [4, 4, 4]), 'FLOAT32': ([1, 0.5, 1, 1, 1, 1, 1, 0.6, 1], [3.5, 4, 3.6]),
}


def gemv(E, op, dtype_name='INT32'):
    """ExampleCppEdsl.GEMV_* and GEMVC_INT64, plaidml/edsl/examples/gemv.cc:14-139: A x + y, and (5 A) x + 4 y
    (answer 19 19 19 on all-ones inputs); plus MaxPool1D on three elements (max_pool_1d.cc:30-35, :65-68)."""
    dt = getattr(E.DType, dtype_name)
    npdt = np.dtype(dtype_name.lower())
    A, x, y = E.Placeholder(dt, [3, 3]), E.Placeholder(dt, [3]), E.Placeholder(dt, [3])
    i, j = E.TensorIndexes(2)
    O = E.Contraction().outShape(3).outAccess(i).sum(A[i, j] * x[j]).build() + y
    i2, j2 = E.TensorIndexes(2)
    O2 = E.Contraction().outShape(3).outAccess(i2).sum((A * 5)[i2, j2] * x[j2]).build() + y * 4
    i3, j3 = E.TensorIndexes(2)
    P = E.Contraction().outShape(1).outAccess(i3).max(y[2 * i3 + j3]).add_constraint(j3 < 2).build()
    a = np.array(GEMV_ANSWERS[dtype_name][0], npdt).reshape(3, 3)
    return E.Program('gemv', [A, x, y], [O, O2, P]), [a, np.ones(3, npdt), np.ones(3, npdt)], EXACT


def funky_sum(E, op):
    """CppEdsl.FunkySum, plaidml/edsl/tests/edsl_test.cc:2709-2719: fractional index polynomial."""
    I = E.Placeholder(E.DType.FLOAT32, [3])
    K = E.Placeholder(E.DType.FLOAT32, [3])
    i, j = E.TensorIndexes(2)
    O = E.Contraction().outShape(5).outAccess(i).sum(I[(i - j + 1) // 2] * K[j]).build()
    return E.Program('funky_sum', [I, K], [O]), [np.array([1, 2, 3], np.float32)] * 2, EXACT


def defract_long(E, op):
    """test_defract_long, plaidml/edsl/tests/edsl_test.py:433-460: transposed-conv style access."""
    shape = [1, 3, 3, 1]
    I = E.Placeholder(E.DType.FLOAT32, shape)
    K = E.Placeholder(E.DType.FLOAT32, shape)
    n, x0, x1, co, ci, k0, k1 = E.TensorIndexes(7)
    O = E.Contraction().outShape(1, 5, 5, 1).outAccess(n, x0, x1, co).sum(
        I[n, (x0 + k0 - 1) // 2, (x1 + k1 - 1) // 2, ci] * K[2 - k0, 2 - k1, co, ci]).build()
    return E.Program('defract_long', [I, K], [O]), [
        np.array([[[[1], [3], [-1]], [[0], [2], [4]], [[1], [-1], [-2]]]], np.float32),
        np.array([[[[2], [3], [4]], [[6], [-3], [-1]], [[-1], [-2], [1]]]], np.float32)], EXACT


def flatten_by_contraction(E, op):
    """`no_reduce` of pmlc/dialect/tile/tests/compute-bounds.mlir:34-45: O[d1 + 10 d0] = I[d0, d1], an output access
    that is a sum of two indices."""
    I = E.Placeholder(E.DType.FLOAT32, [10, 10])
    d0, d1 = E.TensorIndexes(2)
    O = E.Contraction().outShape(100).outAccess(d1 + d0 * 10).assign(I[d0, d1]).build()
    return E.Program('no_reduce', [I], [O]), [_rng(3).standard_normal((10, 10)).astype(np.float32)], EXACT


def scatter_form_transposed_conv(E, op, N=2, H=6, CI=3, CO=4, dtype_name='FLOAT32'):
    """A stride-2 transposed convolution written from the input's point of view: every input pixel (x, y) adds its
    3x3 footprint to O[n, 2x + i - 1, 2y + j - 1, co].  Two output coordinates are sums of indices, many index
    tuples meet in one output element, footprints hang over the border, and the odd output row / column 2H - 1
    ... 2H is reached by one tap only."""
    dt = getattr(E.DType, dtype_name)
    I = E.Placeholder(dt, [N, H, H, CI])
    K = E.Placeholder(dt, [3, 3, CI, CO])
    n, x, y, i, j, ci, co = E.TensorIndexes(7)
    O = E.Contraction().outShape(N, 2 * H, 2 * H, CO).outAccess(n, 2 * x + i - 1, 2 * y + j - 1, co).sum(
        I[n, x, y, ci] * K[i, j, ci, co]).build()
    r = _rng(21)
    vals = [r.integers(-3, 4, (N, H, H, CI)).astype(np.float32), r.integers(-3, 4, (3, 3, CI, CO)).astype(np.float32)]
    return E.Program('scatter_form_transposed_conv', [I, K], [O]), vals, EXACT


def scatter_form_transposed_conv_answer(I, K):
    """The same by explicit loops over the input pixels (float64; the test data are small integers, so exact)."""
    N, H, _, CI = I.shape
    CO = K.shape[3]
    O = np.zeros((N, 2 * H, 2 * H, CO))
    for x in range(H):
        for y in range(H):
            for i in range(3):
                for j in range(3):
                    ox, oy = 2 * x + i - 1, 2 * y + j - 1
                    if 0 <= ox < 2 * H and 0 <= oy < 2 * H:
                        O[:, ox, oy, :] += I[:, x, y, :].astype(np.float64) @ K[i, j].astype(np.float64)
    return O


def mirrored_sum_of_indices(E, op):
    """O[7 - i + 2 j, c] += A[i, c] * B[j, c]: a negative and a non-unit coefficient in one output coordinate (i in
    0..5, j in 0..3), another coordinate plain."""
    A = E.Placeholder(E.DType.INT32, [6, 5])
    B = E.Placeholder(E.DType.INT32, [4, 5])
    i, j, c = E.TensorIndexes(3)
    O = E.Contraction().outShape(14, 5).outAccess(7 - i + 2 * j, c).sum(A[i, c] * B[j, c]).build()
    r = _rng(22)
    return E.Program('mirrored_sum_of_indices', [A, B], [O]), [r.integers(-9, 10, (6, 5)).astype(np.int32),
                                                               r.integers(-9, 10, (4, 5)).astype(np.int32)], EXACT


def max_rows(E, op):
    """CppEdsl.Max, plaidml/edsl/tests/edsl_test.cc:576-590."""
    A = E.Placeholder(E.DType.FLOAT32, [3, 3])
    i, j = E.TensorIndexes(2)
    R = E.Contraction().outShape(3).outAccess(i).max(A[i, j]).build()
    return E.Program('max', [A], [R]), [np.array([-5, -6, -7, 4, 5, 6, 7, 8, 9], np.float32).reshape(3, 3)], EXACT


def use_default(E, op):
    """test_use_default, plaidml/edsl/tests/edsl_test.py:390-406: assign into one slice of an initialised output."""
    P = E.Placeholder(E.DType.FLOAT32, [2, 7, 3, 4])
    I = E.Placeholder(E.DType.FLOAT32, [2, 3, 4])
    b, i1, i2 = E.TensorIndexes(3)
    O = E.Contraction().outShape(2, 7, 3, 4).outAccess(b, 3, i1, i2).init(P).assign(I[b, i1, i2]).build()
    r = _rng(5)
    return E.Program('use_default', [I, P], [O]), [r.standard_normal((2, 3, 4)).astype(np.float32),
                                                   r.standard_normal((2, 7, 3, 4)).astype(np.float32)], EXACT


def eltwise_mix(E, op):
    """Broadcast compare, casts, round and relu in one program (known answers of the single ops:
    plaidml/edsl/tests/edsl_test.cc:158-182, 319-333, 631-643, 1820-1835; quantize.cc:16-32)."""
    A = E.Placeholder(E.DType.FLOAT32, [3, 4])
    B = E.Placeholder(E.DType.FLOAT32, [3, 1])
    C = E.cast(A >= B, E.DType.INT32)
    R = E.round(A * 2.5) + E.cast(C, E.DType.FLOAT32)
    Q = E.cast(E.relu(A - B) * 256.0, E.DType.INT8)
    r = _rng(6)
    return E.Program('eltwise', [A, B], [C, R, Q]), [r.uniform(-0.45, 0.45, (3, 4)).astype(np.float32),
                                                     r.uniform(-0.2, 0.2, (3, 1)).astype(np.float32)], EXACT


def libm_tail_f32(E, op, M=24, N=40, K=16):
    """Float intrinsics as the fused tail of a contraction and with broadcast operands: dot -> sin -> erf,
    pow with a per-column exponent, fmod, tan/atan/sinh chains (single ops pinned by tests/intrinsic_cases.py)."""
    A = E.Placeholder(E.DType.FLOAT32, [M, K])
    B = E.Placeholder(E.DType.FLOAT32, [K, N])
    P = E.Placeholder(E.DType.FLOAT32, [N])
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(M, N).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    S = E.erf(E.sin(C)) + E.cos(C)
    W = E.pow(E.abs(C) + 0.5, P) % 1.5
    T = E.atan(E.sinh(E.tanh(C))) - E.asinh(C) + E.cosh(E.tan(C * 0.1))
    U = E.asin(E.tanh(C)) + E.acos(E.tanh(C)) + E.atanh(E.tanh(C) * 0.5) + E.acosh(E.abs(C) + 1.0)
    r = _rng(21)
    return E.Program('libm_tail', [A, B, P], [S, W, T, U]), [r.uniform(-1, 1, (M, K)).astype(np.float32),
                                                            r.uniform(-1, 1, (K, N)).astype(np.float32),
                                                            r.uniform(0.5, 2.5, (N,)).astype(np.float32)], FP32


def bits_and_truth(E, op):
    """Integer bit operations with mixed widths, broadcasting and immediates, and truth-value operations on
    floats with NaNs (ordered compares: pmlc/conversion/tile_to_linalg/tile_to_linalg.cc:311-370)."""
    A = E.Placeholder(E.DType.INT32, [6, 8])
    B = E.Placeholder(E.DType.INT32, [8])
    Cc = E.Placeholder(E.DType.UINT8, [6, 1])
    F = E.Placeholder(E.DType.FLOAT32, [6, 8])
    X = ((A & B) | (A << 3)) ^ (~B)
    Y = (A >> 2) % 7 + (1 << Cc)
    Z = (Cc >> 1) | 0x80
    L = E.logical_xor(E.logical_and(F, A), E.logical_or(E.logical_not(F), B))
    r = _rng(22)
    f = r.uniform(-1, 1, (6, 8)).astype(np.float32)
    f[r.uniform(size=f.shape) < 0.3] = 0.0
    f[0, 0] = np.nan
    f[1, 3] = -0.0
    a = r.integers(-1000, 1000, (6, 8)).astype(np.int32)
    a[2, 2] = 0
    b = r.integers(-50, 50, (8,)).astype(np.int32)
    b[1] = 0
    return E.Program('bits', [A, B, Cc, F], [X, Y, Z, L]), [a, b, r.integers(0, 8, (6, 1)).astype(np.uint8), f], EXACT


def dot_f16_acc_f32(E, op, M=8, N=32, K=16):
    """CppEdsl.DotF16_AccF32, plaidml/edsl/tests/edsl_test.cc:500-545: half inputs widened, summed in fp32, narrowed
    (the reference compares with tolerance 1e-2 against the same fp32 loop)."""
    A = E.Placeholder(E.DType.FLOAT16, [M, K])
    B = E.Placeholder(E.DType.FLOAT16, [K, N])
    i, j, k = E.TensorIndexes(3)
    C32 = E.Contraction().outShape(M, N).outAccess(i, j).sum(E.cast(A, E.DType.FLOAT32)[i, k] * E.cast(B, E.DType.FLOAT32)[k, j]).build()
    r = _rng(2)
    return E.Program('dot_f16_acc_f32', [A, B], [E.cast(C32, E.DType.FLOAT16)]), [
        r.standard_normal((M, K)).astype(np.float16), r.standard_normal((K, N)).astype(np.float16)], BF16


def row_reductions(E, op, dtype_name='FLOAT32'):
    """Reductions along memory (the shape of a softmax's row max and row sum, a mean, a norm): over the
    innermost axis, over the two innermost axes, into a strided output, onto an initial value, over a
    shifted window, and over rows long enough for a whole workgroup.  Integer types wrap."""
    dt = getattr(E.DType, dtype_name)
    X = E.Placeholder(dt, [6, 5, 200])
    Y = E.Placeholder(dt, [2, 5000])
    P = E.Placeholder(dt, [6, 5])
    i, j, k = E.TensorIndexes(3)
    outs = [
        E.Contraction().outShape(6, 5).outAccess(i, j).sum(X[i, j, k]).build(),
        E.Contraction().outShape(6).outAccess(i).max(X[i, j, k]).build(),
        E.Contraction().outShape(6, 1, 5).outAccess(i, 0, j).min(X[i, j, k]).build(),
        E.Contraction().outShape(6, 5).outAccess(i, j).init(P).sum(X[i, j, k]).build(),
        E.Contraction().outShape(6, 5).outAccess(i, j).sum(X[i, j, k + 3]).build(),
        E.Contraction().outShape(2).outAccess(i).sum(Y[i, k]).build(),
        E.Contraction().outShape(2).outAccess(i).max(Y[i, k]).build(),
        E.Contraction().outShape(5).outAccess(j).sum(X[i, j, k]).build(),  # not along memory: the general kernel
    ]
    r = _rng(31)
    if dtype_name in ('FLOAT32', 'BFLOAT16', 'FLOAT16'):
        outs.append(E.Contraction().outShape(6, 5).outAccess(i, j).product(X[i, j, k]).build())
        vals = [r.uniform(0.97, 1.03, (6, 5, 200)), r.standard_normal((2, 5000)), r.standard_normal((6, 5))]
        vals = [v.astype(np.float32) for v in vals]
        if dtype_name == 'BFLOAT16':
            vals = [_bf16(v) for v in vals]
        elif dtype_name == 'FLOAT16':
            vals = [v.astype(np.float16) for v in vals]
        tol = FP32 if dtype_name == 'FLOAT32' else BF16
    else:
        nd = np.dtype(dtype_name.lower())
        info = np.iinfo(nd)
        vals = [r.integers(info.min, int(info.max) + 1, shape, dtype=nd) for shape in ((6, 5, 200), (2, 5000), (6, 5))]
        tol = EXACT
    return E.Program('row_reductions', [X, Y, P], outs), vals, tol


def float_chains(E, op, dtype_name='FLOAT32', inner=40):
    """Standalone elementwise chains of plain float arithmetic with every kind of second operand: a whole
    tensor, one value per column, one value per row, a single value and an immediate."""
    dt = getattr(E.DType, dtype_name)
    A = E.Placeholder(dt, [6, inner])
    B = E.Placeholder(dt, [6, inner])
    col = E.Placeholder(dt, [inner])
    row = E.Placeholder(dt, [6, 1])
    one = E.Placeholder(dt, [1])
    outs = [
        E.relu(A * B + col) - row,
        E.exp(A - row) / (B * B + 1.5),
        E.tanh(E.sqrt(A * A + 0.25)) * one,
        E.max(A, col) + E.min(B, row) - (-A),
        E.log(A * A + 1.0) / row,
        (2.0 - A) * (3.0 / (B * B + 1.0)),
    ]
    r = _rng(32)
    vals = [r.standard_normal(s).astype(np.float32) for s in ((6, inner), (6, inner), (inner,))]
    vals += [r.uniform(0.5, 2.0, (6, 1)).astype(np.float32), np.array([1.75], np.float32)]
    if dtype_name == 'BFLOAT16':
        vals = [_bf16(v) for v in vals]
    return E.Program('float_chains', [A, B, col, row, one], outs), vals, FP32 if dtype_name == 'FLOAT32' else BF16


def batched_dots(E, op):
    """CppEdsl.HighDimDot / OuterDimDot, plaidml/edsl/tests/edsl_test.cc:418-446: a dot under three batch
    dimensions, once with the contracted dimension innermost and once with it second."""
    M, N, K, X, Y, Z = 8, 32, 16, 5, 4, 4
    A = E.Placeholder(E.DType.FLOAT32, [X, Y, Z, M, K])
    B = E.Placeholder(E.DType.FLOAT32, [X, Y, Z, K, N])
    A2 = E.Placeholder(E.DType.FLOAT32, [X, K, Y, Z, M])
    B2 = E.Placeholder(E.DType.FLOAT32, [X, K, Y, Z, N])
    m, n, k, x, y, z = E.TensorIndexes(6)
    C = E.Contraction().outShape(X, Y, Z, M, N).outAccess(x, y, z, m, n).sum(A[x, y, z, m, k] * B[x, y, z, k, n]).build()
    C2 = E.Contraction().outShape(X, Y, Z, M, N).outAccess(x, y, z, m, n).sum(A2[x, k, y, z, m] * B2[x, k, y, z, n]).build()
    r = _rng(41)
    vals = [r.standard_normal(s).astype(np.float32) for s in ((X, Y, Z, M, K), (X, Y, Z, K, N), (X, K, Y, Z, M), (X, K, Y, Z, N))]
    return E.Program('batched_dots', [A, B, A2, B2], [C, C2]), vals, FP32


def double_dot_dup_out(E, op):
    """CppEdsl.DoubleDot / DupOut, edsl_test.cc:547-563, 1084-1100: dot(dot(A, B), C) returned three times."""
    A = E.Placeholder(E.DType.FLOAT32, [10, 20])
    B = E.Placeholder(E.DType.FLOAT32, [20, 30])
    C = E.Placeholder(E.DType.FLOAT32, [30, 40])
    R = op.dot(op.dot(A, B), C)
    r = _rng(42)
    return E.Program('dup_out', [A, B, C], [R, R, R]), [r.standard_normal(s).astype(np.float32)
                                                        for s in ((10, 20), (20, 30), (30, 40))], FP32


def mnist_mlp(E, op):
    """CppEdsl.MnistMlp, edsl_test.cc:645-662: 784 -> 512 -> 512 -> 10, relu, relu, softmax."""
    f32 = E.DType.FLOAT32
    shapes = [(1, 784), (784, 512), (512,), (512, 512), (512,), (512, 10), (10,)]
    X, K1, b1, K2, b2, K3, b3 = [E.Placeholder(f32, list(s)) for s in shapes]
    d1 = op.relu(op.dot(X, K1) + b1)
    d2 = op.relu(op.dot(d1, K2) + b2)
    Y = op.softmax(op.dot(d2, K3) + b3, 1)
    r = _rng(43)
    vals = [(r.standard_normal(s) * (0.05 if len(s) == 2 and s[0] > 1 else 1.0)).astype(np.float32) for s in shapes]
    return E.Program('mnist_mlp', [X, K1, b1, K2, b2, K3, b3], [Y]), vals, FP32


def mnist_cnn(E, op, side=28):
    """CppEdsl.MnistCnn, edsl_test.cc:664-769, at 28 x 28 (the reference builds it at 224 x 224 and only runs it):
    two SAME 3x3 convolutions written as contractions, the 2x2 max pool with its two constraints, flatten by
    reshape, two dense layers, softmax."""
    f32 = E.DType.FLOAT32

    def conv(I, K):
        N, X0, X1, CI = I.shape if not callable(getattr(I, 'shape', None)) else I.compute_shape().sizes
        K0, K1, _, CO = K.shape if not callable(getattr(K, 'shape', None)) else K.compute_shape().sizes
        n, x0, x1, co, ci, k0, k1 = E.TensorIndexes(7)
        return E.Contraction().outShape(N, X0, X1, CO).outAccess(n, x0, x1, co).sum(
            I[n, x0 + k0 - (K0 // 2), x1 + k1 - (K1 // 2), ci] * K[k0, k1, ci, co]).build()

    def pool(I):
        N, X0, X1, C = I.shape if not callable(getattr(I, 'shape', None)) else I.compute_shape().sizes
        n, x0, x1, i, j, c = E.TensorIndexes(6)
        return E.Contraction().outShape(N, (X0 + 1) // 2, (X1 + 1) // 2, C).outAccess(n, x0, x1, c).max(
            I[n, 2 * x0 + i, 2 * x1 + j, c]).add_constraint(i < 2).add_constraint(j < 2).build()

    flat = (side // 2) * (side // 2) * 64
    shapes = [(1, side, side, 1), (3, 3, 1, 32), (32,), (3, 3, 32, 64), (64,), (flat, 128), (128,), (128, 100), (100,)]
    X, K1, b1, K2, b2, K3, b3, K4, b4 = [E.Placeholder(f32, list(s)) for s in shapes]
    c1 = op.relu(conv(X, K1) + b1)
    c2 = op.relu(conv(c1, K2) + b2)
    p1 = pool(c2)
    fl = E.reshape(p1, [1, flat])
    d1 = op.relu(op.dot(fl, K3) + b3)
    Y = op.softmax(op.dot(d1, K4) + b4, 1)
    r = _rng(44)
    vals = [(r.standard_normal(s) * (0.1 if len(s) > 1 and s != shapes[0] else 1.0)).astype(np.float32) for s in shapes]
    vals[5] = (vals[5] * 0.1).astype(np.float32)
    return E.Program('mnist_cnn', [X, K1, b1, K2, b2, K3, b3, K4, b4], [Y]), vals, FP32


def lars_momentum4d(E, op):
    """CppEdsl.LarsMomentum4d, edsl_test.cc:796-830: two whole-tensor norms (contractions into a scalar) steer an
    elementwise update; the learning rate is a rank-0 input."""
    f32 = E.DType.FLOAT32
    shape = [4, 7, 3, 9]
    X, G, V = [E.Placeholder(f32, shape) for _ in range(3)]
    LR = E.Placeholder(f32, [])

    def norm(T):
        idxs = E.TensorIndexes(4)
        return E.sqrt(E.Contraction().sum((T * T)[idxs]).build())

    coeff, decay, momentum = 1. / 1024., 1. / 2048., 1. / 8.
    xn, gn = norm(X), norm(G)
    loc = LR * coeff * xn / (gn + decay * xn)
    nv = momentum * V + loc * (G + decay * X)
    r = _rng(45)
    vals = [r.standard_normal(shape).astype(np.float32) for _ in range(3)] + [np.array(0.5, np.float32)]
    return E.Program('lars_momentum4d', [X, G, V, LR], [X - nv, nv]), vals, FP32


def repeat_and_global_min(E, op):
    """CppEdsl.RepeatElements (edsl_test.cc:856-875: out[n0, 3 n1 + k, n2] = in[n0, n1, n2], k < 3), GlobalMin
    (:895-907: -max(-I) over everything) and UniqueNames (:877-893: two inputs share a name)."""
    f32 = E.DType.FLOAT32
    I = E.Placeholder(f32, [10, 10, 10])
    n0, n1, n2, k = E.TensorIndexes(4)
    O = E.Contraction().outShape(10, 30, 10).outAccess(n0, 3 * n1 + k, n2).assign(I[n0, n1, n2]).add_constraint(k < 3).build()
    i, j, l = E.TensorIndexes(3)
    M = -(E.Contraction().max((-I)[i, j, l]).build())
    A, B = E.Placeholder(f32, [1], name='A'), E.Placeholder(f32, [1], name='B')
    C0, C1 = E.Placeholder(f32, [1], name='C'), E.Placeholder(f32, [1], name='C')
    r = _rng(46)
    vals = [r.standard_normal((10, 10, 10)).astype(np.float32)] + [np.array([v], np.float32) for v in (1, 2, 4, 8)]
    return E.Program('repeat_min_names', [I, A, B, C0, C1], [O, M, A + B + C0 + C1]), vals, EXACT


def python_front_end_cases(E, op):
    """The small cases of plaidml/edsl/tests/edsl_test.py: test_cast_scalar (:265, a rank-0 input), test_cast_folder
    (:271, a cast to the same type), test_funky_names (:462, a program name that is no identifier), test_identity and
    test_two_outputs (:482, :513: an input returned as is, twice), test_trace (:573)."""
    S = E.Placeholder(E.DType.INT32, [])
    V = E.Placeholder(E.DType.INT32, [3])
    I = E.Placeholder(E.DType.FLOAT32, [3], name='I')
    K = E.Placeholder(E.DType.FLOAT32, [3], name='K')
    i, j = E.TensorIndexes(2)
    F = E.Contraction().outShape(5).outAccess(i).sum(I[(i - j + 1) // 2] * K[j]).build()
    outs = [E.cast(S, E.DType.FLOAT32), E.cast(V, E.DType.INT32), F, I, I, E.trace(K, 'msg')]
    vals = [np.array(3, np.int32), np.array([1, 2, 3], np.int32), np.array([1, 2, 3], np.float32), np.array([1, 2, 3], np.float32)]
    return E.Program('this-is-not an identifier', [S, V, I, K], outs), vals, EXACT


def python_conv_cases(E, op):
    """test_conv_1d (:277), test_conv_2d_dilated (:284), test_complex_conv_2d (:291, grouped, strided, dilated,
    SAME_LOWER; its first spatial access reads x1 where x0 is meant, and so does this restatement) and test_lens
    (:578, the same convolution written through NHWC/HWCK and NCHW/CKHW lenses), at reduced image sizes."""
    f32 = E.DType.FLOAT32

    def conv_1d(I, K):
        N, X, KX, CI, CO = E.TensorDims(5)
        n, x, k, ci, co = E.TensorIndexes(5)
        I.bind_dims(N, X, CI)
        K.bind_dims(KX, CI, CO)
        return E.Contraction().outShape(N, X - KX + 1, CO).outAccess(n, x, co).sum(I[n, x + k, ci] * K[k, ci, co]).build()

    def conv_2d_dilated(I, K):
        N, X, Y, KX, KY, CI, CO = E.TensorDims(7)
        n, x, y, kx, ky, ci, co = E.TensorIndexes(7)
        I.bind_dims(N, X, Y, CI)
        K.bind_dims(KX, KY, CI, CO)
        return E.Contraction().outShape(N, X - 2 * (KX - 1), Y - 3 * (KY - 1), CO).outAccess(n, x, y, co).sum(
            I[n, x + 2 * kx, y + 3 * ky, ci] * K[kx, ky, ci, co]).build()

    def complex_conv_2d(I, K, s0, s1, d0, d1):
        N, G, GCI, GCO, X0, X1, K0, K1 = E.TensorDims(8)
        n, g, gci, gco, x0, x1, k0, k1 = E.TensorIndexes(8)
        I.bind_dims(N, X0, X1, G, GCI)
        K.bind_dims(K0, K1, G, GCI, GCO)
        Y0, Y1 = (X0 + s0 - 1) // s0, (X1 + s1 - 1) // s1
        EK0, EK1 = d0 * (K0 - 1) + 1, d1 * (K1 - 1) + 1
        P0, P1 = ((Y0 - 1) * s0 + EK0 - X0) // 2, ((Y1 - 1) * s1 + EK1 - X1) // 2
        return E.Contraction().outShape(N, Y0, Y1, G, GCO).outAccess(n, x0, x1, g, gco).sum(
            I[n, s0 * x1 + d0 * k0 - P0, s1 * x1 + d1 * k1 - P1, g, gci] * K[k0, k1, g, gci, gco]).build()

    def conv_2d(I, K, I_layout, K_layout):
        I_lens, K_lens = E.TensorLens(I_layout, 'NHWC'), E.TensorLens(K_layout, 'HWCK')
        I, K = I.use(I_lens), K.use(K_lens)
        CI, CO, K0, K1, N, X0, X1 = E.TensorDims(7)
        n, x0, x1, k0, k1, ci, co = E.TensorIndexes(7)
        I.bind_dims(N, X0, X1, CI)
        K.bind_dims(K0, K1, CI, CO)
        return E.Contraction(I_lens).outShape(N, X0 - (K0 - 1), X1 - (K1 - 1), CO).outAccess(n, x0, x1, co).sum(
            I[n, x0 + k0 - (K0 // 2), x1 + k1 - (K1 // 2), ci] * K[k0, k1, ci, co]).build()

    shapes = [(1, 24, 3), (3, 3, 1), (1, 20, 22, 1), (3, 3, 1, 8), (1, 12, 14, 3, 3), (3, 3, 3, 3, 8), (1, 1, 1, 1, 1),
              (1, 1, 1, 1, 1), (1, 12, 12, 3), (3, 3, 3, 8), (1, 3, 12, 12), (3, 8, 5, 5)]
    P = [E.Placeholder(f32, list(s)) for s in shapes]
    outs = [conv_1d(P[0], P[1]), conv_2d_dilated(P[2], P[3]), complex_conv_2d(P[4], P[5], 1, 2, 1, 2),
            complex_conv_2d(P[6], P[7], 1, 2, 1, 2), conv_2d(P[8], P[9], 'NHWC', 'HWCK'), conv_2d(P[10], P[11], 'NCHW', 'CKHW')]
    r = _rng(47)
    return E.Program('python_convs', P, outs), [r.standard_normal(s).astype(np.float32) for s in shapes], FP32


def u64_add(E, op):
    """CppEdsl.Add, plaidml/edsl/tests/edsl_test.cc:335-374 (64-bit integer elementwise)."""
    A = E.Placeholder(E.DType.UINT64, [3, 3])
    B = E.Placeholder(E.DType.UINT64, [3, 3])
    a = [1, 2, 3, 4, 5, 6 + (1 << 12), 7 + (1 << 24), 8 + (1 << 32), 9 + (1 << 40)]
    b = [1, 2 + (1 << 12), 3, 4 + (1 << 24), 5, 6 + (1 << 32), 7, 8 + (1 << 40), 9]
    return E.Program('add', [A, B], [A + B]), [np.array(a, np.uint64).reshape(3, 3), np.array(b, np.uint64).reshape(3, 3)], EXACT


def higher_precision_constants(E, op):
    """CppEdsl.HigherPrecisionConstants, plaidml/edsl/tests/edsl_test.cc:140-156."""
    A = E.Placeholder(E.DType.FLOAT32, [3, 3])
    C = A + E.cast(E.Constant(1), E.DType.UINT64) + E.cast(E.Constant(2.0), E.DType.FLOAT64)
    return E.Program('hpc', [A], [C]), [np.arange(1, 10, dtype=np.float32).reshape(3, 3)], EXACT


# ---- the five workload configurations, reduced ---------------------------------------------------------


def eq_combination(E, op):
    """The `eq` combination (plaidml/edsl/edsl.h:421, result type i1: pmlc/ast/eval.cc:25; lowered as a compare
    aggregated in one-bit arithmetic: tile_to_linalg.cc:1257-1262, :485-544).  any / all / parity of matches per
    output point, integer comparands and mixed float / integer ones, one output with uncovered elements."""
    r = _rng(31)
    a = r.integers(0, 3, (6, 8)).astype(np.int32)
    b = r.integers(0, 3, (8, 5)).astype(np.int32)
    f = r.integers(0, 3, (6, 8)).astype(np.float32)
    f[0, 0] = np.nan
    A = E.Placeholder(E.DType.INT32, a.shape)
    B = E.Placeholder(E.DType.INT32, b.shape)
    F = E.Placeholder(E.DType.FLOAT32, f.shape)
    outs = []
    for agg in ('max', 'min', 'sum', 'product'):
        i, j, k = E.TensorIndexes(3)
        outs.append(getattr(E.Contraction().outShape(6, 5).outAccess(i, j), agg)(A[i, k] == B[k, j]).build())
    i, j, k = E.TensorIndexes(3)
    outs.append(E.Contraction().outShape(6, 5).outAccess(i, j).sum(F[i, k] == B[k, j]).build())
    i, j, k = E.TensorIndexes(3)
    outs.append(E.Contraction().outShape(7, 6).outAccess(i, j).min(A[i, k] == B[k, j]).build())
    return E.Program('eq_combination', [A, B, F], outs), [a, b, f], EXACT


def eq_combination_answers(a, b, f):
    """What the mathematics fixes for eq_combination: numpy any / all / parity of the match table."""
    m = a[:, :, None] == b[None, :, :]
    mf = f[:, :, None] == b[None, :, :].astype(np.float32)
    part = np.ones((7, 6), bool)   # elements the contraction never reaches keep min's identity: true
    part[:6, :5] = m.all(1)
    return [m.any(1), m.all(1), (m.sum(1) % 2).astype(bool), m.all(1), (mf.sum(1) % 2).astype(bool), part]


def partial_cover_gemm(E, op):
    """A matrix product that writes only part of its result (a larger outShape, a shifted outAccess): the
    rest holds the aggregation identity, also under a fused elementwise tail (exp(0) = 1)."""
    r = _rng(32)
    a = r.standard_normal((8, 16)).astype(np.float32) * 0.25
    b = r.standard_normal((16, 8)).astype(np.float32) * 0.25
    A = E.Placeholder(E.DType.FLOAT32, a.shape)
    B = E.Placeholder(E.DType.FLOAT32, b.shape)
    outs = []
    for shape, dj in (((16, 8), 0), ((16, 12), 0), ((8, 12), 4)):
        i, j, k = E.TensorIndexes(3)
        outs.append(E.exp(E.Contraction().outShape(*shape).outAccess(i, j + dj).sum(A[i, k] * B[k, j]).build()))
    return E.Program('partial_cover_gemm', [A, B], outs), [a, b], FP32


def broadcast_first_min_max(E, op):
    """maximum / minimum / select-as-max whose first operand is the broadcast one (X[8] against Y[4,8])."""
    r = _rng(33)
    x = r.standard_normal(8).astype(np.float32)
    y = r.standard_normal((4, 8)).astype(np.float32)
    y[1, 2] = np.nan
    x[5] = np.nan
    X = E.Placeholder(E.DType.FLOAT32, x.shape)
    Y = E.Placeholder(E.DType.FLOAT32, y.shape)
    outs = [op.maximum(X, Y), op.minimum(X, Y), E.select(X < Y, Y, X), E.select(X > Y, X, Y),
            op.maximum(Y, X), op.minimum(Y, X)]
    return E.Program('broadcast_first_min_max', [X, Y], outs), [x, y], FP32



def bf16_rounding_placement(E, op):
    """bf16 contractions accumulate in fp32 and round once, to nearest even, after the last tap and after the
    initial value went in.  Integer-valued inputs whose exact sums fp32 holds and bf16 does not:
    256 + 1 + 1 + 1 = 259 -> 260 (rounding after every tap gives 256, after pairs 258);
    2 (initial value) + 256 + 1 = 259 -> 260 (rounding the sum before the initial value goes in gives 258);
    columns 1: 128 + 0.5 + 0.5 + 0.5 = 129.5 -> 130 (per tap: 128)."""
    a = np.array([[256, 1, 1, 1], [128, 0.5, 0.5, 0.5]], np.float32)
    b = np.ones((4, 2), np.float32)
    a2 = np.array([[256, 1, 0, 0]], np.float32)
    c = np.full((1, 2), 2, np.float32)
    A = E.Placeholder(E.DType.BFLOAT16, a.shape)
    B = E.Placeholder(E.DType.BFLOAT16, b.shape)
    A2 = E.Placeholder(E.DType.BFLOAT16, a2.shape)
    C = E.Placeholder(E.DType.BFLOAT16, c.shape)
    i, j, k = E.TensorIndexes(3)
    O = E.Contraction().outShape(2, 2).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    i, j, k = E.TensorIndexes(3)
    O2 = E.Contraction().outShape(1, 2).outAccess(i, j).sum(A2[i, k] * B[k, j]).init(C).build()
    i, j, k = E.TensorIndexes(3)
    O3 = E.Contraction().outShape(1, 2).outAccess(i, j).sum(A2[i, k] * B[k, j]).build() + C
    # the same sums at a size the matrix-core kernels take: rows of 256, 1, 1, 1, 0 ... and 128, .5, .5, .5, 0 ...
    a4 = np.zeros((64, 64), np.float32)
    a4[0::2, :4] = a[0]
    a4[1::2, 20:24] = a[1]
    c4 = np.zeros((64, 64), np.float32)
    c4[:, 1::2] = 2
    a4[2, 3] = 0  # row 2 with the initial value 2: 2 + 256 + 1 + 1 = 260 exactly; without: 258
    A4 = E.Placeholder(E.DType.BFLOAT16, a4.shape)
    B4 = E.Placeholder(E.DType.BFLOAT16, [64, 64])
    C4 = E.Placeholder(E.DType.BFLOAT16, c4.shape)
    i, j, k = E.TensorIndexes(3)
    O4 = E.Contraction().outShape(64, 64).outAccess(i, j).sum(A4[i, k] * B4[k, j]).build()
    O5 = O4 + C4
    return (E.Program('bf16_rounding_placement', [A, B, A2, C, A4, B4, C4], [O, O2, O3, O4, O5]),
            [a, b, a2, c, a4, np.ones((64, 64), np.float32), c4], EXACT)


def _bf16_rounding_answers():
    o4 = np.zeros((64, 64), np.float32)
    o4[0::2] = 260
    o4[1::2] = 130
    o4[2] = 258
    o5 = o4.copy()
    o5[0::2, 1::2] = 262   # 2 + 259 = 261 -> 262 (tie to even; 260 + 2 after an early rounding is 262 as well)
    o5[1::2, 1::2] = 132   # 2 + 129.5 = 131.5 -> 132 (130 + 2 = 132 as well)
    o5[2, 1::2] = 260      # 2 + 258 = 260 exactly
    return [np.array([[260, 260], [130, 130]], np.float32), np.array([[260, 260]], np.float32),
            np.array([[260, 260]], np.float32), o4, o5]


BF16_ROUNDING_ANSWERS = _bf16_rounding_answers()

def config0_gemm_f32(E, op, n=128, seed=1):
    """configs[0]: C[M,N] += A[M,K] * B[K,N], fp32, U(-1,1)."""
    A = E.Placeholder(E.DType.FLOAT32, [n, n])
    B = E.Placeholder(E.DType.FLOAT32, [n, n])
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(n, n).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    r = _rng(seed)
    return E.Program('gemm_f32', [A, B], [C]), [r.uniform(-1, 1, (n, n)).astype(np.float32),
                                                r.uniform(-1, 1, (n, n)).astype(np.float32)], FP32


def config1_conv(E, op, dtype_name='BFLOAT16', N=2, H=14, W=14, CI=64, CO=64):
    """configs[1]: relu(conv2d(I, F) + B), NHWC, 3x3, stride 1, SAME."""
    dt = getattr(E.DType, dtype_name)
    I = E.Placeholder(dt, [N, H, W, CI])
    F = E.Placeholder(dt, [3, 3, CI, CO])
    B = E.Placeholder(dt, [CO])
    O = op.relu(op.convolution(I, F) + B)
    r = _rng(2)
    Iv = r.standard_normal((N, H, W, CI)).astype(np.float32)
    Fv = (_rng(3).standard_normal((3, 3, CI, CO)) * np.sqrt(2.0 / (9 * CI))).astype(np.float32)
    Bv = (_rng(4).standard_normal(CO) * 0.1).astype(np.float32)
    if dtype_name == 'BFLOAT16':
        Iv, Fv, Bv = _bf16(Iv), _bf16(Fv), _bf16(Bv)
    return E.Program('conv', [I, F, B], [O]), [Iv, Fv, Bv], BF16 if dtype_name == 'BFLOAT16' else FP32


def config2_int8_gemm(E, op, M=64, N=48, K=32):
    """configs[2]: int8 x int8 -> int32 (cast before the contraction, plaidml/edsl/tests/edsl_test.cc:509-545
    pattern), then Q = cast(round(clip(cast(C, f32) * S, -127, 127)), int8) with S per output column."""
    A = E.Placeholder(E.DType.INT8, [M, K])
    B = E.Placeholder(E.DType.INT8, [K, N])
    S = E.Placeholder(E.DType.FLOAT32, [N])
    Ai, Bi = E.cast(A, E.DType.INT32), E.cast(B, E.DType.INT32)
    i, j, k = E.TensorIndexes(3)
    C = E.Contraction().outShape(M, N).outAccess(i, j).sum(Ai[i, k] * Bi[k, j]).build()
    Q = E.cast(E.round(op.clip(E.cast(C, E.DType.FLOAT32) * S, -127.0, 127.0)), E.DType.INT8)
    r4, r5, r6 = _rng(4), _rng(5), _rng(6)
    return E.Program('int8_gemm', [A, B, S], [C, Q]), [r4.integers(-127, 128, (M, K), dtype=np.int8),
                                                       r5.integers(-127, 128, (K, N), dtype=np.int8),
                                                       r6.uniform(0.001, 0.01, N).astype(np.float32)], EXACT


def config3_xception_block(E, op, N=2, H=19, W=19, C=32, dtype_name='BFLOAT16', with_pool_input=False):
    """configs[3]: depthwise 3x3 -> pointwise 1x1 -> scale/shift + ReLU -> maxpool 3x3/2 with window argmax."""
    dt = getattr(E.DType, dtype_name)
    I = E.Placeholder(dt, [N, H, W, C])
    Fdw = E.Placeholder(dt, [3, 3, C, 1])
    Fpw = E.Placeholder(dt, [1, 1, C, C])
    scale = E.Placeholder(dt, [C])
    shift = E.Placeholder(dt, [C])
    D = op.convolution(I, Fdw, depthwise=True)
    P = op.convolution(D, Fpw)
    R = op.relu(P * scale + shift)
    M = op.pool(R, 'max', [3, 3], [2, 2], autopad=op.SAME_UPPER)
    n, x0, x1, c, k0, k1 = E.TensorIndexes(6)
    IX = E.index([3, 3], 0) * 3 + E.index([3, 3], 1)
    AM = E.Contraction().outShape(M.shape).outAccess(n, x0, x1, c).max(
        E.cond(R[n, 2 * x0 + k0 - 1, 2 * x1 + k1 - 1, c], M[n, x0, x1, c], IX[k0, k1])).build()
    Iv = _rng(7).standard_normal((N, H, W, C)).astype(np.float32)
    Fd = (_rng(8).standard_normal((3, 3, C, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    Fp = (_rng(9).standard_normal((1, 1, C, C)) * np.sqrt(2.0 / C)).astype(np.float32)
    sc = _rng(10).uniform(0.5, 1.5, C).astype(np.float32)
    sh = _rng(11).uniform(-0.5, 0.5, C).astype(np.float32)
    vals = [Iv, Fd, Fp, sc, sh]
    if dtype_name == 'BFLOAT16':
        vals = [_bf16(v) for v in vals]
    outs = [M, AM, R] if with_pool_input else [M, AM]
    return E.Program('xception_block', [I, Fdw, Fpw, scale, shift], outs), vals, BF16 if dtype_name == 'BFLOAT16' else FP32


def window_argmax_of(R, M):
    """The window argmax of config3_xception_block worked out in numpy from the pool's own input R and result M:
    the largest tap number 3 * k0 + k1 whose element equals the window maximum (taps outside the image never
    match), 0 where none does."""
    N, H, W, C = R.shape
    OH, OW = M.shape[1], M.shape[2]
    padded = np.full((N, 2 * OH + 1, 2 * OW + 1, C), np.nan, np.float32)  # NaN never equals
    padded[:, 1:H + 1, 1:W + 1] = R
    best = np.zeros(M.shape, np.int32)
    for k0 in range(3):
        for k1 in range(3):
            tap = padded[:, k0:k0 + 2 * OH:2, k1:k1 + 2 * OW:2]
            best = np.where(tap == M, np.int32(3 * k0 + k1), best)
    return best


def classifier_tail(E, op, N=4, C=64, K=10, dtype_name='FLOAT32'):
    """The tail of configs[4]: global average pool -> dense + bias -> softmax."""
    dt = getattr(E.DType, dtype_name)
    X = E.Placeholder(dt, [N, 7, 7, C])
    Wt = E.Placeholder(dt, [C, K])
    b = E.Placeholder(dt, [K])
    G = op.mean(X, [1, 2])
    L = op.dot(G, Wt) + b
    Y = op.softmax(L, 1)
    vals = [_rng(20).standard_normal((N, 7, 7, C)).astype(np.float32),
            (_rng(21).standard_normal((C, K)) * 0.2).astype(np.float32), np.zeros(K, np.float32)]
    if dtype_name == 'BFLOAT16':
        vals = [_bf16(v) for v in vals]
    return E.Program('tail', [X, Wt, b], [Y, op.argmax(L, 1)]), vals, BF16 if dtype_name == 'BFLOAT16' else FP32


def residual_block(E, op, N=2, H=8, C=64, dtype_name='BFLOAT16'):
    """One ResNet bottleneck-style residual: relu(conv1x1(relu(conv3x3(x) + b1)) + b2 + x), weights as constants."""
    dt = getattr(E.DType, dtype_name)
    f1 = (_rng(30).standard_normal((3, 3, C, C)) * np.sqrt(2.0 / (9 * C))).astype(np.float32)
    f2 = (_rng(31).standard_normal((1, 1, C, C)) * np.sqrt(2.0 / C)).astype(np.float32)
    b1 = (_rng(32).standard_normal(C) * 0.1).astype(np.float32)
    b2 = (_rng(33).standard_normal(C) * 0.1).astype(np.float32)
    xv = _rng(34).standard_normal((N, H, H, C)).astype(np.float32)
    if dtype_name == 'BFLOAT16':
        f1, f2, b1, b2, xv = (_bf16(v) for v in (f1, f2, b1, b2, xv))
    X = E.Placeholder(dt, [N, H, H, C])
    F1, F2, B1, B2 = (E.Constant(v, dt) for v in (f1, f2, b1, b2))
    Y = op.relu(op.convolution(X, F1) + B1)
    Z = op.relu(op.convolution(Y, F2) + B2 + X)
    return E.Program('residual', [X], [Z]), [xv], BF16 if dtype_name == 'BFLOAT16' else FP32


def toy_parallel_conv(E, op):
    """The reference benchmark tool's `toy_parallel_conv` network with its own weights and input
    (plaidbench/plaidbench/networks/keras/toy_parallel_conv.py:18-41), fp32: conv 7x7/2 SAME 3->64 + ReLU, then
    relu(relu(conv 1x1/2 64->256) + relu(conv 3x3/2 SAME 64->256)).  Returns the program, its inputs (the 224x224x3
    image first, then weights and biases) and the golden fixture (tests/golden/toy_parallel_conv.npz)."""
    import os
    fx = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), 'golden', 'toy_parallel_conv.npz'))
    f32 = E.DType.FLOAT32
    image = np.repeat(np.repeat(fx['image'][None].astype(np.float32), 7, axis=1), 7, axis=2)  # values 0..255, unscaled
    X = E.Placeholder(f32, list(image.shape))
    ins, vals = [X], [image]

    def conv(x, i, stride):
        W = E.Placeholder(f32, list(fx['kernel%d' % i].shape))
        B = E.Placeholder(f32, list(fx['bias%d' % i].shape))
        ins.extend([W, B])
        vals.extend([fx['kernel%d' % i], fx['bias%d' % i]])
        return op.relu(op.convolution(x, W, strides=[stride, stride], autopad=op.SAME_UPPER) + B)

    l1 = conv(X, 1, 2)
    out = op.relu(conv(l1, 2, 2) + conv(l1, 3, 2))
    return E.Program('toy_parallel_conv', ins, [out]), vals, fx


def resnet50_tiny(E, op):
    """The full ResNet-50 v1.5 topology (plaidml_amd/resnet50.py) at 1/4 width on 2 x 32x32 images."""
    from plaidml_amd import resnet50
    from oracle.tile_oracle import round_bf16
    prog, _, _ = resnet50.build(E, op, batch=2, image=32, classes=10, dtype_name='BFLOAT16', base=16, round_fn=round_bf16)
    x = _bf16(_rng(11).uniform(0, 1, (2, 32, 32, 3)).astype(np.float32))
    return prog, [x], BF16


ALL = {
    'dot_f32': dot_f32,
    'gemm_int32': lambda E, op: gemm_int(E, op, 'INT32'),
    'gemm_int64': lambda E, op: gemm_int(E, op, 'INT64'),
    'gemm_uint64': lambda E, op: gemm_int(E, op, 'UINT64'),
    'gemm_int8': lambda E, op: gemm_int(E, op, 'INT8'),
    'gemv_int64': lambda E, op: gemv(E, op, 'INT64'),
    'gemv_uint64': lambda E, op: gemv(E, op, 'UINT64'),
    'gemv_int32': lambda E, op: gemv(E, op, 'INT32'),
    'gemv_int8': lambda E, op: gemv(E, op, 'INT8'),
    'gemv_float32': lambda E, op: gemv(E, op, 'FLOAT32'),
    'funky_sum': funky_sum,
    'defract_long': defract_long,
    'flatten_by_contraction': flatten_by_contraction,
    'scatter_form_transposed_conv': scatter_form_transposed_conv,
    'mirrored_sum_of_indices': mirrored_sum_of_indices,
    'max_rows': max_rows,
    'use_default': use_default,
    'eltwise_mix': eltwise_mix,
    'libm_tail_f32': libm_tail_f32,
    'dot_f16_acc_f32': dot_f16_acc_f32,
    'bits_and_truth': bits_and_truth,
    'row_reductions_f32': row_reductions,
    'row_reductions_bf16': lambda E, op: row_reductions(E, op, 'BFLOAT16'),
    'row_reductions_f16': lambda E, op: row_reductions(E, op, 'FLOAT16'),
    'row_reductions_int32': lambda E, op: row_reductions(E, op, 'INT32'),
    'row_reductions_uint8': lambda E, op: row_reductions(E, op, 'UINT8'),
    'row_reductions_int16': lambda E, op: row_reductions(E, op, 'INT16'),
    'float_chains_f32': float_chains,
    'float_chains_bf16': lambda E, op: float_chains(E, op, 'BFLOAT16'),
    'float_chains_f32_ragged': lambda E, op: float_chains(E, op, 'FLOAT32', inner=37),
    'batched_dots': batched_dots,
    'double_dot_dup_out': double_dot_dup_out,
    'mnist_mlp': mnist_mlp,
    'mnist_cnn': mnist_cnn,
    'lars_momentum4d': lars_momentum4d,
    'repeat_and_global_min': repeat_and_global_min,
    'python_front_end_cases': python_front_end_cases,
    'python_conv_cases': python_conv_cases,
    'u64_add': u64_add,
    'higher_precision_constants': higher_precision_constants,
    'eq_combination': eq_combination,
    'partial_cover_gemm': partial_cover_gemm,
    'broadcast_first_min_max': broadcast_first_min_max,
    'bf16_rounding_placement': bf16_rounding_placement,
    'config0_gemm_f32': config0_gemm_f32,
    'config1_conv_bf16': lambda E, op: config1_conv(E, op, 'BFLOAT16'),
    'config1_conv_f32': lambda E, op: config1_conv(E, op, 'FLOAT32', CI=32, CO=48),
    'config2_int8_gemm': config2_int8_gemm,
    'config3_xception_block_bf16': config3_xception_block,
    'config3_xception_block_f32': lambda E, op: config3_xception_block(E, op, C=16, dtype_name='FLOAT32'),
    'classifier_tail_f32': classifier_tail,
    # one image: the batch index has a single value and is folded out of every access before kernels are matched
    'single_image_xception_block_f32': lambda E, op: config3_xception_block(E, op, N=1, C=16, dtype_name='FLOAT32'),
    'single_image_classifier_tail_f32': lambda E, op: classifier_tail(E, op, N=1),
    # 136 fp32 channels are 544 bytes per pixel: the depthwise result feeding the pointwise product is laid out at a
    # pitch of whole 128-byte lines (640 bytes)
    'xception_block_f32_pitched_temporary': lambda E, op: config3_xception_block(E, op, N=1, C=136, dtype_name='FLOAT32'),
    'residual_block_bf16': residual_block,
    'resnet50_tiny_bf16': resnet50_tiny,
}

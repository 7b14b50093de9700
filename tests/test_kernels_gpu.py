"""Parity of the HIP kernel library (called through its C ABI) against the CPU oracle.

Bars: bit-exact for int8 -> int32 and for index outputs; rtol 1e-3 for fp32;
rtol 2e-2 for bf16 (both taken from the north-star statement of this build).
"""
import ctypes

import numpy as np
import pytest

from oracle import tile_oracle as E
from oracle import tile_oplib as op
from plaidml_amd import hipkernels as hk

pytestmark = pytest.mark.gpu

D = E.DType
FP32_RTOL, BF16_RTOL = 1e-3, 2e-2


@pytest.fixture(scope='module', autouse=True)
def _device():
    hk.init(0)
    print('device:', hk.device_name(), flush=True)


def bf16(a):
    return E.bf16_bits(np.asarray(a, np.float32))


# schedule bits (hk.flag_tile / hk.flag_conv) that a test adds to every descriptor run_gemm / run_conv build
FORCED = {'flags': 0}


def run_gemm(A, B, in_dt, out_dt, init=None, init_strides=(0, 0), init_dt=0, tail=None, operands=(), c_dt=None,
             extra_out=None, flags=0, invokes=1):
    M, K = A.shape
    _, N = B.shape
    d = hk.GemmDesc()
    d.in_dtype, d.out_dtype = in_dt, out_dt
    d.flags = flags | FORCED['flags']
    d.m, d.n, d.k = M, N, K
    d.lda, d.ldb, d.ldc = K, N, N
    d.c_dtype = c_dt if c_dt is not None else out_dt
    if init is not None:
        d.init_kind, d.init_dtype = 1, init_dt
        d.init_row_stride, d.init_col_stride = init_strides
    if tail is not None:
        d.tail = tail
    plan = hk.lib().pml_hip_gemm_dispatch(ctypes.byref(d))
    assert plan, hk.lib().pml_hip_last_error()
    print('plan:', hk.describe(plan), flush=True)
    dA, dB = hk.DeviceBuffer.from_numpy(A), hk.DeviceBuffer.from_numpy(B)
    np_c = {hk.F32: np.float32, hk.BF16: np.uint16, hk.I32: np.int32, hk.I8: np.int8}[d.c_dtype]
    dC = hk.DeviceBuffer(M * N * np.dtype(np_c).itemsize)
    dI = hk.DeviceBuffer.from_numpy(init) if init is not None else None
    dops = [hk.DeviceBuffer.from_numpy(o) for o in operands]
    outs = []
    dX = None
    if extra_out is not None:
        dX = hk.DeviceBuffer(M * N * np.dtype(extra_out).itemsize)
        outs = [dX.ptr]
    for _ in range(invokes):  # (the last run's result is the one returned: what a run leaves behind must not show in the next)
        hk.check(hk.lib().pml_hip_fill_u32(dC.ptr, 0xdeadbeef, M * N * np.dtype(np_c).itemsize // 4, None))
        hk.check(hk.lib().pml_hip_gemm_invoke(plan, dA.ptr, dB.ptr, dC.ptr, dI.ptr if dI else None,
                                              hk.ptr_array([o.ptr for o in dops]), hk.ptr_array(outs), None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    C = dC.to_numpy(np_c, (M, N))
    X = dX.to_numpy(extra_out, (M, N)) if dX else None
    hk.lib().pml_hip_plan_free(plan)
    return (C, X) if extra_out is not None else C


@pytest.mark.parametrize('M,N,K', [(1024, 1024, 1024), (96, 80, 40), (8, 16, 32), (257, 130, 68)])
def test_gemm_f32(M, N, K):
    rng = np.random.default_rng(1)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    C = run_gemm(A, B, hk.F32, hk.F32)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(C, ref, rtol=FP32_RTOL, atol=1e-4)


def test_gemm_f32_matches_oracle_contraction():
    rng = np.random.default_rng(2)
    Av = rng.standard_normal((8, 32)).astype(np.float32)
    Bv = rng.standard_normal((32, 16)).astype(np.float32)
    A, B = E.Placeholder(D.FLOAT32, Av.shape), E.Placeholder(D.FLOAT32, Bv.shape)
    i, j, k = E.TensorIndexes(3)
    O = E.Contraction().outShape(8, 16).outAccess(i, j).sum(A[i, k] * B[k, j]).build()
    ref, = E.run(E.Program('dot', [A, B], [O]), [Av, Bv])
    np.testing.assert_allclose(run_gemm(Av, Bv, hk.F32, hk.F32), ref, rtol=FP32_RTOL, atol=1e-5)


TILE_NAMES = ['64x64', '128x64', '128x128', '128x64w8', '128x128w8', '128x128w8s2', '256x128w16', '64x64w8k2', '256x256w8', '128x64n2', '192x384w8', '64x64ks']


@pytest.mark.parametrize('tile', TILE_NAMES)
def test_every_tile_configuration(tile, monkeypatch):
    """Every tiling the library holds (named in the descriptor's schedule bits), on a problem that is ragged
    in M, N and K and spans several tiles: int8 bit for bit, bf16 (+ bias + relu, the direct tail where the tile is
    interior) and fp32 against float64."""
    monkeypatch.setitem(FORCED, 'flags', hk.flag_tile(tile))
    print('tile', tile, flush=True)
    rng = np.random.default_rng(7)
    M, N, K = 600, 520, 336
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    np.testing.assert_array_equal(run_gemm(A, B, hk.I8, hk.I32), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.int32))
    # rows of whole 16-byte vectors: the int8 right-hand side is read where it lies, through transposing LDS reads
    B16 = rng.integers(-127, 128, (K, 528), dtype=np.int8)
    np.testing.assert_array_equal(run_gemm(A, B16, hk.I8, hk.I32), (A.astype(np.int64) @ B16.astype(np.int64)).astype(np.int32))
    Af = E.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    Bf = E.round_bf16(rng.standard_normal((K, N)).astype(np.float32))
    bias = E.round_bf16(rng.standard_normal(N).astype(np.float32))
    tail = hk.make_tail(ops=[(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)])
    C = E.bf16_from_bits(run_gemm(bf16(Af), bf16(Bf), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail))
    ref = np.maximum(Af.astype(np.float64) @ Bf.astype(np.float64) + bias, 0)
    np.testing.assert_allclose(C, ref, rtol=BF16_RTOL, atol=BF16_RTOL * np.sqrt(K))
    A32 = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B32 = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    np.testing.assert_allclose(run_gemm(A32, B32, hk.F32, hk.F32), A32.astype(np.float64) @ B32.astype(np.float64),
                               rtol=FP32_RTOL, atol=1e-3)
    np.testing.assert_allclose(run_gemm(A32, B32, hk.F32, hk.F32, flags=hk.FP32_AS_BF16X3),
                               A32.astype(np.float64) @ B32.astype(np.float64), rtol=FP32_RTOL, atol=1e-3)


@pytest.mark.parametrize('M,N,K', [(1024, 1024, 1024), (257, 130, 68), (256, 384, 4096)])
def test_gemm_f32_as_three_bf16_products(M, N, K):
    """fp32 operands split into bf16 head + remainder in registers, three bf16 MFMAs per term.  U(-1, 1) operands make
    every result a sum of K terms of both signs (K = 4096: results of size ~21 from terms of size ~1/3), the case
    where a lost low part shows; the bar is fp32's own (rtol 1e-3).  What the split drops is bounded as well: the
    largest deviation from float64 stays below 4 x 2^-16 x sqrt(K) x E|ab|."""
    rng = np.random.default_rng(41)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    bias = rng.standard_normal(N).astype(np.float32)
    tail = hk.make_tail(ops=[(hk.EPI_RELU, hk.F32, 0, 0, 0.0)])
    C = run_gemm(A, B, hk.F32, hk.F32, init=bias, init_strides=(0, 1), init_dt=hk.F32, tail=tail, flags=hk.FP32_AS_BF16X3)
    ref = np.maximum(A.astype(np.float64) @ B.astype(np.float64) + bias, 0)
    np.testing.assert_allclose(C, ref, rtol=FP32_RTOL, atol=1e-3)
    assert np.abs(C - ref).max() < 4 * 2.0 ** -16 * np.sqrt(K) * 0.25 + 1e-5
    # values a bf16 holds exactly go through unchanged: small integers give the exact integer result
    Ai = rng.integers(-8, 9, (M, K)).astype(np.float32)
    Bi = rng.integers(-8, 9, (K, N)).astype(np.float32)
    np.testing.assert_array_equal(run_gemm(Ai, Bi, hk.F32, hk.F32, flags=hk.FP32_AS_BF16X3), Ai @ Bi)


@pytest.mark.parametrize('long_k', [False, True])
@pytest.mark.parametrize('stride', [0, 2])
def test_gemm_two_products(stride, long_k):
    """C = relu(A.B + b + A2.B2 + b2) in one launch: the second left-hand side as plain rows, and as the pixel rows a
    1x1 convolution with stride 2 reads from an NHWC image (a residual block's projection shortcut).  With few tiles and
    long K's (the shortcut of a network's last stage at batch 1) the slabs of both products are shared out among
    workgroups; a split then begins in the middle of the first product or in the second."""
    rng = np.random.default_rng(21)
    NB, OH, OW, K1, K2, N = (1, 7, 7, 520, 1024, 136) if long_k else (3, 7, 9, 72, 40, 136)
    M = NB * OH * OW
    A = E.round_bf16(rng.standard_normal((M, K1)).astype(np.float32))
    B = E.round_bf16(rng.standard_normal((K1, N)).astype(np.float32) * (0.2 if not long_k else 0.05))
    B2 = E.round_bf16(rng.standard_normal((K2, N)).astype(np.float32) * (0.2 if not long_k else 0.05))
    b1 = E.round_bf16(rng.standard_normal(N).astype(np.float32))
    b2 = E.round_bf16(rng.standard_normal(N).astype(np.float32))
    if stride:
        H2, W2 = (OH - 1) * stride + 2, (OW - 1) * stride + 1
        img = E.round_bf16(rng.standard_normal((NB, H2, W2, K2)).astype(np.float32))
        A2 = img[:, :(OH - 1) * stride + 1:stride, :(OW - 1) * stride + 1:stride].reshape(M, K2)
        a2_dev = img
    else:
        A2 = E.round_bf16(rng.standard_normal((M, K2)).astype(np.float32))
        a2_dev = A2
    d = hk.GemmDesc()
    d.in_dtype = d.out_dtype = d.c_dtype = hk.BF16
    d.m, d.n, d.k, d.lda, d.ldb, d.ldc = M, N, K1, K1, N, N
    d.init_kind, d.init_dtype, d.init_row_stride, d.init_col_stride = 1, hk.BF16, 0, 1
    d.tail = hk.make_tail(ops=[(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)])
    d.k2, d.lda2, d.ldb2, d.init2_kind = K2, K2, N, 1
    if stride:
        d.a2_stride, d.a2_h, d.a2_w, d.a2_oh, d.a2_ow = stride, H2, W2, OH, OW
    L = hk.lib()
    plan = L.pml_hip_gemm_dispatch(ctypes.byref(d))
    assert plan, L.pml_hip_last_error()
    print('plan:', hk.describe(plan), flush=True)
    assert ('K split over workgroups' in hk.describe(plan)) == long_k
    bufs = [hk.DeviceBuffer.from_numpy(bf16(x)) for x in (A, B, b1, a2_dev, B2, b2)]
    dC = hk.DeviceBuffer(M * N * 2)
    none = hk.ptr_array([])
    # the plain entry point refuses a plan with a second product
    assert L.pml_hip_gemm_invoke(plan, bufs[0].ptr, bufs[1].ptr, dC.ptr, bufs[2].ptr, none, none, None) != 0
    hk.check(L.pml_hip_gemm_pack_b2(plan, bufs[4].ptr, None))
    hk.check(L.pml_hip_gemm_invoke2(plan, bufs[0].ptr, bufs[1].ptr, dC.ptr, bufs[2].ptr, bufs[3].ptr, None, bufs[5].ptr, none, none, None))
    hk.check(L.pml_hip_stream_sync(None))
    C = E.bf16_from_bits(dC.to_numpy(np.uint16, (M, N)))
    ref = np.maximum(A.astype(np.float64) @ B + A2.astype(np.float64) @ B2 + b1 + b2, 0)
    np.testing.assert_allclose(C, ref, rtol=BF16_RTOL, atol=BF16_RTOL if not long_k else 4e-2)
    L.pml_hip_plan_free(plan)


@pytest.mark.parametrize('tile', ['', '128x128w8s2', '128x64w8', '256x128w16', '256x256w8'])
def test_gemm_bf16_step_tails_bit_exact(tile, monkeypatch):
    """The bf16 tails that leave the accumulators directly (interior tiles) and through LDS (the ragged last column
    tile) must round alike: small-integer operands make the fp32 accumulation exact, so the expected result is
    fixed bit for bit by the declared step semantics -- each step rounds to bf16 -- for the folded batch
    normalisation relu(x * scale + shift) and for relu(x + residual)."""
    rng = np.random.default_rng(33)
    M, N, K = 300, 392, 72
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    bias = E.round_bf16(rng.standard_normal(N).astype(np.float32) * 8)
    scale = E.round_bf16(rng.uniform(0.5, 1.5, N).astype(np.float32))
    shift = E.round_bf16(rng.standard_normal(N).astype(np.float32) * 20)
    res = E.round_bf16(rng.standard_normal((M, N)).astype(np.float32) * 30)
    x = E.round_bf16((A @ B + bias).astype(np.float32))  # exact sum, one rounding
    for relu in (False, True):
        ops = [(hk.EPI_MUL, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 1, 0.0)]
        ops += [(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)] if relu else []
        tail = hk.make_tail(ops=ops, operands=[(hk.BF16, 0, 1), (hk.BF16, 0, 1)])
        C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail,
                     operands=(bf16(scale), bf16(shift)))
        want = E.round_bf16(E.round_bf16(x * scale) + shift)
        want = np.maximum(want, 0) if relu else want
        np.testing.assert_array_equal(C, bf16(want))
        ops = [(hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 0, 0.0)] + ([(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)] if relu else [])
        tail = hk.make_tail(ops=ops, operands=[(hk.BF16, N, 1)])
        C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail,
                     operands=(bf16(res),))
        want = E.round_bf16(x + res)
        want = np.maximum(want, 0) if relu else want
        np.testing.assert_array_equal(C, bf16(want))


def test_gemm_random_shapes_all_kinds():
    """Forty seeded random problems -- ragged M, N, K, every element kind, the tails with a vector path (none, bias + relu,
    + residual + relu, scale / shift + relu) -- against float64 / exact integer arithmetic; bf16 results additionally
    bit for bit against the step semantics where the accumulation is exact (small-integer operands)."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        kind = ['f32', 'bf16', 'i8', 'f32x3'][case % 4]
        M, N = int(rng.integers(1, 700)), int(rng.integers(1, 90)) * 8
        K = int(rng.integers(1, 60)) * (16 if kind == 'i8' else 8)
        tail_kind = ['none', 'relu', 'residual', 'scale_shift'][int(rng.integers(0, 4))]
        print('case', case, kind, (M, N, K), tail_kind, flush=True)
        if kind == 'i8':
            A = rng.integers(-127, 128, (M, K), dtype=np.int8)
            B = rng.integers(-127, 128, (K, N), dtype=np.int8)
            np.testing.assert_array_equal(run_gemm(A, B, hk.I8, hk.I32), (A.astype(np.int64) @ B.astype(np.int64)).astype(np.int32))
            continue
        dt = hk.BF16 if kind == 'bf16' else hk.F32
        flags = hk.FP32_AS_BF16X3 if kind == 'f32x3' else 0
        if kind == 'bf16':   # small integers: the fp32 accumulation is exact, every rounding is pinned
            A = rng.integers(-4, 5, (M, K)).astype(np.float32)
            B = rng.integers(-4, 5, (K, N)).astype(np.float32)
        else:
            A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
            B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
        rnd = E.round_bf16 if kind == 'bf16' else (lambda x: np.asarray(x, np.float32))
        enc = bf16 if kind == 'bf16' else (lambda x: np.asarray(x, np.float32))
        bias = rnd(rng.standard_normal(N).astype(np.float32) * 4)
        scale = rnd(rng.uniform(0.5, 1.5, N).astype(np.float32))
        shift = rnd(rng.standard_normal(N).astype(np.float32) * 8)
        res = rnd(rng.standard_normal((M, N)).astype(np.float32) * 16)
        relu = [(hk.EPI_RELU, dt, 0, 0, 0.0)]
        x64 = A.astype(np.float64) @ B.astype(np.float64)
        if tail_kind == 'none':
            C = run_gemm(enc(A), enc(B), dt, dt, flags=flags)
            want = rnd(x64.astype(np.float32)) if kind == 'bf16' else x64
        elif tail_kind == 'relu':
            C = run_gemm(enc(A), enc(B), dt, dt, init=enc(bias), init_strides=(0, 1), init_dt=dt, tail=hk.make_tail(ops=relu), flags=flags)
            want = np.maximum(rnd((x64 + bias).astype(np.float32)) if kind == 'bf16' else x64 + bias, 0)
        elif tail_kind == 'residual':
            tail = hk.make_tail(ops=[(hk.EPI_ADD, dt, hk.OPND_TENSOR, 0, 0.0)] + relu, operands=[(dt, N, 1)])
            C = run_gemm(enc(A), enc(B), dt, dt, init=enc(bias), init_strides=(0, 1), init_dt=dt, tail=tail, operands=(enc(res),), flags=flags)
            want = np.maximum(rnd(rnd((x64 + bias).astype(np.float32)) + res) if kind == 'bf16' else x64 + bias + res, 0)
        else:
            tail = hk.make_tail(ops=[(hk.EPI_MUL, dt, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_ADD, dt, hk.OPND_TENSOR, 1, 0.0)] + relu,
                                operands=[(dt, 0, 1), (dt, 0, 1)])
            C = run_gemm(enc(A), enc(B), dt, dt, init=enc(bias), init_strides=(0, 1), init_dt=dt, tail=tail,
                         operands=(enc(scale), enc(shift)), flags=flags)
            if kind == 'bf16':
                want = np.maximum(rnd(rnd(rnd((x64 + bias).astype(np.float32)) * scale) + shift), 0)
            else:
                want = np.maximum((x64 + bias) * scale + shift, 0)
        if kind == 'bf16':
            np.testing.assert_array_equal(C, bf16(want), err_msg='case %d' % case)
        else:
            np.testing.assert_allclose(C, want, rtol=FP32_RTOL, atol=1e-3, err_msg='case %d' % case)


def test_gemm_bf16_4096_sampled():
    """bf16 4096^3 with N(0,1) inputs (the large-tile path): sampled rows and columns against float64."""
    rng = np.random.default_rng(9)
    n = 4096
    A = E.round_bf16(rng.standard_normal((n, n)).astype(np.float32))
    B = E.round_bf16(rng.standard_normal((n, n)).astype(np.float32))
    C = E.bf16_from_bits(run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16))
    rows = rng.choice(n, 16, replace=False)
    ref = A[rows].astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(C[rows], ref, rtol=BF16_RTOL, atol=BF16_RTOL * 64)   # results are ~N(0, 64^2)
    cols = rng.choice(n, 16, replace=False)
    np.testing.assert_allclose(C[:, cols], A.astype(np.float64) @ B[:, cols].astype(np.float64), rtol=BF16_RTOL, atol=BF16_RTOL * 64)


@pytest.mark.parametrize('M,N,K', [(512, 512, 512), (100, 72, 48), (4096, 4096, 4096)])
def test_gemm_i8_bit_exact(M, N, K):
    rng = np.random.default_rng(4)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    C = run_gemm(A, B, hk.I8, hk.I32)
    # |acc| <= K * 127^2 < 2^31, so the int32 result equals the exact integer product
    if M * N * K <= 1 << 27:
        ref = A.astype(np.int64) @ B.astype(np.int64)
        np.testing.assert_array_equal(C, ref.astype(np.int32))
    else:
        # full size: exact check on sampled rows / columns, and the checksum identity sum_j C[i,j] = A[i,:] . rowsum(B)
        rows = rng.choice(M, 24, replace=False)
        ref = A[rows].astype(np.int64) @ B.astype(np.int64)
        np.testing.assert_array_equal(C[rows], ref.astype(np.int32))
        cols = rng.choice(N, 24, replace=False)
        refc = A.astype(np.int64) @ B[:, cols].astype(np.int64)
        np.testing.assert_array_equal(C[:, cols], refc.astype(np.int32))
        lhs = C.astype(np.int64).sum(axis=1)
        rhs = A.astype(np.int64) @ B.astype(np.int64).sum(axis=1)
        np.testing.assert_array_equal(lhs, rhs)


def test_gemm_i8_requantize_tail():
    # C = A.B (si32, stored to the extra output); Q = cast(round(clip(cast(C, f32) * S[col], -127, 127)), si8)
    rng = np.random.default_rng(5)
    M, N, K = 128, 96, 64
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    S = rng.uniform(0.001, 0.01, N).astype(np.float32)
    tail = hk.make_tail(
        ops=[(hk.EPI_STORE, hk.I32, 0, 0, 0.0), (hk.EPI_CAST, hk.F32, 0, 0, 0.0),
             (hk.EPI_MUL, hk.F32, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_MAX, hk.F32, hk.OPND_IMM, 0, -127.0),
             (hk.EPI_MIN, hk.F32, hk.OPND_IMM, 0, 127.0), (hk.EPI_ROUND, hk.F32, 0, 0, 0.0),
             (hk.EPI_CAST, hk.I8, 0, 0, 0.0)],
        operands=[(hk.F32, 0, 1)])
    Q, C = run_gemm(A, B, hk.I8, hk.I32, tail=tail, operands=[S], c_dt=hk.I8, extra_out=np.int32)
    ref = (A.astype(np.int64) @ B.astype(np.int64)).astype(np.int32)
    np.testing.assert_array_equal(C, ref)
    # oracle program for the epilogue
    Cp = E.Placeholder(D.INT32, ref.shape)
    Sp = E.Placeholder(D.FLOAT32, [N])
    x = E.cast(Cp, D.FLOAT32) * Sp
    x = E.select(x < -127.0, E.cast(E.Constant(-127.0), D.FLOAT32), x)
    x = E.select(x < 127.0, x, E.cast(E.Constant(127.0), D.FLOAT32))
    Qo, = E.run(E.Program('q', [Cp, Sp], [E.cast(E.round(x), D.INT8)]), [ref, S])
    np.testing.assert_array_equal(Q, Qo)


@pytest.mark.parametrize('M,N,K', [(49, 512, 2048), (196, 256, 2048), (100, 130, 4096), (1, 1000, 2048), (300, 72, 2064)])
def test_gemm_k_split_over_workgroups(M, N, K, capsys):
    """Few result tiles and a long K: the library shares the K loop out among workgroups (partial tiles in a workspace,
    added up by a second launch that runs the tail; three runs of one plan over the same workspace).  int8 bit for bit -- the sum of the parts is the sum; bf16 with
    bias + residual + relu, fp32 and the split fp32 kind against float64; ragged M, N (a workspace pitch of whole
    vectors) and a K that leaves the last split short."""
    rng = np.random.default_rng(123)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    bias_i = rng.integers(-1000, 1000, N, dtype=np.int32)
    C = run_gemm(A, B, hk.I8, hk.I32, init=bias_i, init_strides=(0, 1), init_dt=hk.I32, invokes=3)
    assert 'K split over workgroups' in capsys.readouterr().out
    np.testing.assert_array_equal(C, (A.astype(np.int64) @ B.astype(np.int64) + bias_i).astype(np.int32))
    Af = E.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    Bf = E.round_bf16((rng.standard_normal((K, N)) / np.sqrt(K)).astype(np.float32))
    bias = E.round_bf16(rng.standard_normal(N).astype(np.float32))
    R = E.round_bf16(rng.standard_normal((M, N)).astype(np.float32))
    tail = hk.make_tail(ops=[(hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_RELU, hk.BF16, 0, 0, 0.0)], operands=[(hk.BF16, N, 1)])
    got = E.bf16_from_bits(run_gemm(bf16(Af), bf16(Bf), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16,
                                    tail=tail, operands=[bf16(R)]))
    assert 'K split over workgroups' in capsys.readouterr().out
    ref = np.maximum(E.round_bf16((Af.astype(np.float64) @ Bf.astype(np.float64) + bias).astype(np.float32)).astype(np.float64) + R, 0)
    np.testing.assert_allclose(got, ref, rtol=BF16_RTOL, atol=2e-2)
    A32 = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B32 = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    for flags in (0, hk.FP32_AS_BF16X3):
        got = run_gemm(A32, B32, hk.F32, hk.F32, flags=flags)
        assert 'K split over workgroups' in capsys.readouterr().out
        np.testing.assert_allclose(got, A32.astype(np.float64) @ B32.astype(np.float64), rtol=FP32_RTOL, atol=2e-3)


@pytest.mark.parametrize('kind', ['bf16', 'f32'])
@pytest.mark.parametrize('shape,k,co,stride', [((1, 7, 7, 512), 3, 512, 1), ((1, 14, 14, 256), 3, 256, 2), ((2, 9, 11, 96), 5, 40, 1)])
def test_conv_k_split_over_workgroups(kind, shape, k, co, stride, capsys):
    """The same for convolutions (the 3x3 layers of a network's last stages at batch 1): a split begins in the middle
    of the tap sequence, also in the middle of a tap's channels (96 channels: one and a half slabs per tap in bf16)."""
    Iv, Fv = _conv_case(kind, shape, k, k, co, op.SAME_UPPER, 57)
    bias = np.random.default_rng(58).standard_normal(co).astype(np.float32)
    if kind == 'bf16':
        bias = E.round_bf16(bias)
        out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, stride=stride, bias=bf16(bias), relu=True))
        ref = oracle_conv(Iv, Fv, D.BFLOAT16, stride, op.SAME_UPPER, bias, True)
        tol = dict(rtol=BF16_RTOL, atol=2e-2)
    else:
        out = run_conv(Iv, Fv, hk.F32, hk.F32, stride=stride, bias=bias, relu=True)
        ref = oracle_conv(Iv, Fv, D.FLOAT32, stride, op.SAME_UPPER, bias, True)
        tol = dict(rtol=FP32_RTOL, atol=1e-3)
    assert 'K split over workgroups' in capsys.readouterr().out
    np.testing.assert_allclose(out, ref, **tol)


def _requant_reference(C32, S, lo, hi):
    """The chain step by step in float32, as the steps are defined: cast, multiply, v > lo ? v : lo, v < hi ? v : hi,
    round half away from zero, truncate to si32, wrap to si8."""
    with np.errstate(invalid='ignore', over='ignore'):
        v = C32.astype(np.float32) * S.astype(np.float32)
        v = np.where(v > np.float32(lo), v, np.float32(lo))
        v = np.where(v < np.float32(hi), v, np.float32(hi))
        r = np.where(v >= 0, np.floor(v + np.float32(0.5)), np.ceil(v - np.float32(0.5)))
        return r.astype(np.int32).astype(np.int8)


@pytest.mark.parametrize('tile', ['64x64', '128x128', '128x128w8s2', '256x128w16', '256x256w8'])
@pytest.mark.parametrize('store,vector_scale', [(True, True), (False, True), (True, False)])
def test_gemm_i8_requantisation_chain_as_straight_code(tile, store, vector_scale, monkeypatch, capsys):
    """The chain a clip-and-round requantisation compiles to -- (store si32)? cast f32, * scale, maxgt lo, min hi, round,
    cast si8 -- runs as straight code behind the int8 GEMM on every tile, the 256x256 one included: both outputs bit for
    bit against the steps evaluated one by one in float32.  Scales of 0.5 / 0.25 put many products exactly half way
    between integers (both signs); one column scale is NaN, one infinite, one negative; a bias is added to the sums."""
    monkeypatch.setitem(FORCED, 'flags', hk.flag_tile(tile))
    rng = np.random.default_rng(77)
    M, N, K = 600, 520, 336
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    B = rng.integers(-127, 128, (K, N), dtype=np.int8)
    A[:40] = rng.integers(-3, 4, (40, K), dtype=np.int8)  # small sums: the clamps do not hide the rounding
    bias = rng.integers(-50, 50, N, dtype=np.int32)
    if vector_scale:
        S = rng.uniform(0.001, 0.01, N).astype(np.float32)
        S[::7], S[1::7] = 0.5, 0.25
        S[3], S[11], S[19] = np.nan, np.inf, -0.004
    else:
        S = np.array([0.5], np.float32)
    ops = ([(hk.EPI_STORE, hk.I32, 0, 0, 0.0)] if store else []) + [
        (hk.EPI_CAST, hk.F32, 0, 0, 0.0), (hk.EPI_MUL, hk.F32, hk.OPND_TENSOR, 0, 0.0),
        (hk.EPI_MAX_GT, hk.F32, hk.OPND_IMM, 0, -127.0), (hk.EPI_MIN, hk.F32, hk.OPND_IMM, 0, 127.0),
        (hk.EPI_ROUND, hk.F32, 0, 0, 0.0), (hk.EPI_CAST, hk.I8, 0, 0, 0.0)]
    tail = hk.make_tail(ops=ops, operands=[(hk.F32, 0, 1 if vector_scale else 0)])
    got = run_gemm(A, B, hk.I8, hk.I32, init=bias, init_strides=(0, 1), init_dt=hk.I32, tail=tail, operands=[S], c_dt=hk.I8,
                   extra_out=np.int32 if store else None)
    assert tile.split('w')[0] in capsys.readouterr().out
    Q, C = got if store else (got, None)
    ref = (A.astype(np.int64) @ B.astype(np.int64) + bias).astype(np.int32)
    if store:
        np.testing.assert_array_equal(C, ref)
    np.testing.assert_array_equal(Q, _requant_reference(ref, S if vector_scale else np.full(N, S[0], np.float32), -127.0, 127.0))


@pytest.mark.parametrize('M,N,K', [(256, 256, 256), (72, 200, 136)])
def test_gemm_bf16(M, N, K):
    rng = np.random.default_rng(6)
    A = E.round_bf16(rng.standard_normal((M, K)).astype(np.float32))
    B = E.round_bf16(rng.standard_normal((K, N)).astype(np.float32))
    C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16)
    ref = E.round_bf16((A.astype(np.float64) @ B.astype(np.float64)).astype(np.float32))
    np.testing.assert_allclose(E.bf16_from_bits(C), ref, rtol=BF16_RTOL, atol=1e-2)


def run_conv(I, F, in_dt, out_dt, stride=1, pad=None, autopad=op.SAME_UPPER, bias=None, relu=False, tail=None,
             operands=(), flags=0, packed=False):
    N, H, W, CI = I.shape
    KH, KW, _, CO = F.shape
    ph, OH = op.compute_padding_and_output_size(H, KH, stride, autopad)
    pw, OW = op.compute_padding_and_output_size(W, KW, stride, autopad)
    if pad is not None:  # explicit symmetric padding
        ph = pw = pad
        OH, OW = (H + 2 * pad - KH) // stride + 1, (W + 2 * pad - KW) // stride + 1
    d = hk.Conv2dDesc()
    d.in_dtype, d.out_dtype, d.c_dtype = in_dt, out_dt, out_dt
    d.flags = flags | FORCED['flags']
    d.n, d.h, d.w, d.ci, d.kh, d.kw, d.co, d.oh, d.ow = N, H, W, CI, KH, KW, CO, OH, OW
    d.stride_h = d.stride_w = stride
    d.dil_h = d.dil_w = 1
    d.pad_h, d.pad_w = ph, pw
    if bias is not None:
        d.init_kind, d.init_dtype = 1, out_dt
        d.init_row_stride, d.init_col_stride = 0, 1
    if tail is not None:
        d.tail = tail
    elif relu:
        d.tail = hk.make_tail(ops=[(hk.EPI_RELU, out_dt, 0, 0, 0.0)])
    plan = hk.lib().pml_hip_conv2d_dispatch(ctypes.byref(d))
    assert plan, hk.lib().pml_hip_last_error()
    print('plan:', hk.describe(plan), flush=True)
    dI, dF = hk.DeviceBuffer.from_numpy(I), hk.DeviceBuffer.from_numpy(F)
    np_c = {hk.F32: np.float32, hk.BF16: np.uint16, hk.I32: np.int32}[out_dt]
    dO = hk.DeviceBuffer(N * OH * OW * CO * np.dtype(np_c).itemsize)
    dB = hk.DeviceBuffer.from_numpy(bias) if bias is not None else None
    dops = [hk.DeviceBuffer.from_numpy(o) for o in operands]
    if packed:  # a constant filter: re-laid once, the invoke is given none
        hk.check(hk.lib().pml_hip_conv2d_pack_filter(plan, dF.ptr, None))
    hk.check(hk.lib().pml_hip_conv2d_invoke(plan, dI.ptr, None if packed else dF.ptr, dO.ptr, dB.ptr if dB else None,
                                            hk.ptr_array([o.ptr for o in dops]), hk.ptr_array([]), None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    out = dO.to_numpy(np_c, (N, OH, OW, CO))
    hk.lib().pml_hip_plan_free(plan)
    return out


def oracle_conv(Iv, Fv, dt, stride, autopad, bias=None, relu=False, pad=None):
    I, F = E.Placeholder(dt, Iv.shape), E.Placeholder(dt, Fv.shape)
    ins, vals = [I, F], [Iv, Fv]
    if pad is not None:
        O = op.convolution(I, F, strides=[stride, stride], autopad=op.EXPLICIT, manual_padding=[pad, pad])
    else:
        O = op.convolution(I, F, strides=[stride, stride], autopad=autopad)
    if bias is not None:
        B = E.Placeholder(dt, bias.shape)
        ins.append(B)
        vals.append(bias)
        O = O + B
    if relu:
        O = op.relu(O)
    out, = E.run(E.Program('conv', ins, [O]), vals)
    return out


@pytest.mark.parametrize('shape,k,stride,autopad', [((2, 12, 12, 32), 3, 1, op.SAME_UPPER), ((1, 9, 11, 64), 3, 2, op.SAME_UPPER),
                                                     ((2, 8, 8, 32), 1, 1, op.VALID), ((1, 14, 14, 32), 7, 2, op.SAME_UPPER)])
@pytest.mark.parametrize('flags', [0, hk.FP32_AS_BF16X3])
def test_conv_f32(shape, k, stride, autopad, flags):
    rng = np.random.default_rng(7)
    Iv = rng.standard_normal(shape).astype(np.float32)
    Fv = (rng.standard_normal((k, k, shape[3], 48)) * 0.1).astype(np.float32)
    bias = rng.standard_normal(48).astype(np.float32)
    out = run_conv(Iv, Fv, hk.F32, hk.F32, stride=stride, autopad=autopad, bias=bias, relu=True, flags=flags)
    ref = oracle_conv(Iv, Fv, D.FLOAT32, stride, autopad, bias, True)
    np.testing.assert_allclose(out, ref, rtol=FP32_RTOL, atol=1e-4)


def test_conv_f32_as_three_bf16_products_configs1_sampled():
    """BASELINE configs[1] in fp32 at full size with the operands split into bf16 head + remainder: sampled pixels
    against float64."""
    rng = np.random.default_rng(2)
    N, H, W, CI, CO = 128, 56, 56, 64, 64
    Iv = rng.standard_normal((N, H, W, CI)).astype(np.float32)
    Fv = (np.random.default_rng(3).standard_normal((3, 3, CI, CO)) * np.sqrt(2.0 / (9 * CI))).astype(np.float32)
    bias = rng.standard_normal(CO).astype(np.float32)
    out = run_conv(Iv, Fv, hk.F32, hk.F32, bias=bias, relu=True, flags=hk.FP32_AS_BF16X3)
    Ip = np.pad(Iv, ((0, 0), (1, 1), (1, 1), (0, 0))).astype(np.float64)
    for _ in range(200):
        n, y, x = rng.integers(N), rng.integers(H), rng.integers(W)
        ref = np.maximum(np.einsum('yxc,yxck->k', Ip[n, y:y + 3, x:x + 3], Fv.astype(np.float64)) + bias, 0)
        np.testing.assert_allclose(out[n, y, x], ref, rtol=FP32_RTOL, atol=1e-4)


@pytest.mark.parametrize('shape,k,stride,co', [((2, 14, 14, 64), 3, 1, 64), ((1, 10, 10, 128), 1, 2, 72), ((2, 7, 9, 64), 3, 2, 40)])
def test_conv_bf16(shape, k, stride, co):
    rng = np.random.default_rng(8)
    Iv = E.round_bf16(rng.standard_normal(shape).astype(np.float32))
    Fv = E.round_bf16((rng.standard_normal((k, k, shape[3], co)) * np.sqrt(2.0 / (k * k * shape[3]))).astype(np.float32))
    bias = E.round_bf16(rng.standard_normal(co).astype(np.float32))
    out = run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, stride=stride, bias=bf16(bias), relu=True)
    ref = oracle_conv(Iv, Fv, D.BFLOAT16, stride, op.SAME_UPPER, bias, True)
    np.testing.assert_allclose(E.bf16_from_bits(out), ref, rtol=BF16_RTOL, atol=1e-2)


def test_conv_random_shapes_all_kinds():
    """Twenty-four seeded random convolutions (1x1 / 3x3 / 5x5, stride 1 / 2, SAME and VALID windows, channel counts that
    do and do not fill 128-byte pixels, bias + ReLU) in fp32, bf16 and split fp32 against the oracle."""
    rng = np.random.default_rng(777)
    for case in range(24):
        kind = ['f32', 'bf16', 'f32x3'][case % 3]
        k = int(rng.choice([1, 3, 3, 5]))
        stride = int(rng.choice([1, 1, 2]))
        ci, co = int(rng.choice([8, 16, 32, 64, 72])), int(rng.choice([8, 24, 64, 96]))
        shape = (int(rng.integers(1, 4)), int(rng.integers(k, 20)), int(rng.integers(k, 24)), ci)
        autopad = op.SAME_UPPER if rng.integers(0, 2) else op.VALID
        print('case', case, kind, shape, 'k', k, 'stride', stride, 'co', co, 'autopad', autopad, flush=True)
        Iv, Fv = _conv_case('bf16' if kind == 'bf16' else 'f32', shape, k, k, co, autopad, 1000 + case)
        bias = rng.standard_normal(co).astype(np.float32)
        if kind == 'bf16':
            bias = E.round_bf16(bias)
            out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, stride=stride, autopad=autopad, bias=bf16(bias), relu=True))
            ref = oracle_conv(Iv, Fv, D.BFLOAT16, stride, autopad, bias, True)
            np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2, err_msg='case %d' % case)
        else:
            out = run_conv(Iv, Fv, hk.F32, hk.F32, stride=stride, autopad=autopad, bias=bias, relu=True,
                           flags=hk.FP32_AS_BF16X3 if kind == 'f32x3' else 0)
            ref = oracle_conv(Iv, Fv, D.FLOAT32, stride, autopad, bias, True)
            np.testing.assert_allclose(out, ref, rtol=FP32_RTOL, atol=1e-4, err_msg='case %d' % case)


def test_conv_bf16_full_size_properties():
    # BASELINE configs[1] at full size: N128 56x56x64 (*) 3x3x64x64 SAME + bias + ReLU, bf16.
    # Size-independent checks: (a) sampled output pixels against a float64 evaluation of the
    # definition, (b) linearity in the filter: conv(I, F1 + F2) = conv(I, F1) + conv(I, F2) up to rounding.
    rng = np.random.default_rng(2)
    Iv = E.round_bf16(rng.standard_normal((128, 56, 56, 64)).astype(np.float32))
    Fv = E.round_bf16((np.random.default_rng(3).standard_normal((3, 3, 64, 64)) * np.sqrt(2.0 / 576)).astype(np.float32))
    bias = np.zeros(64, np.float32)
    out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bf16(bias), relu=True))
    assert out.shape == (128, 56, 56, 64) and (out >= 0).all()
    Ip = np.pad(Iv.astype(np.float64), ((0, 0), (1, 1), (1, 1), (0, 0)))
    F64 = Fv.astype(np.float64)
    pts = [(0, 0, 0), (127, 55, 55), (5, 0, 55), (77, 55, 0)] + [tuple(rng.integers(0, s) for s in (128, 56, 56)) for _ in range(60)]
    for n, y, x in pts:
        win = Ip[n, y:y + 3, x:x + 3, :]
        ref = np.maximum(np.einsum('abc,abcd->d', win, F64), 0)
        np.testing.assert_allclose(out[n, y, x], ref, rtol=BF16_RTOL, atol=2e-2)


def _conv_case(kind, shape, kh, kw, co, autopad, seed):
    rng = np.random.default_rng(seed)
    if kind == 'i8':
        Iv = rng.integers(-127, 128, shape, dtype=np.int8)
        Fv = rng.integers(-127, 128, (kh, kw, shape[3], co), dtype=np.int8)
        return Iv, Fv
    Iv = rng.standard_normal(shape).astype(np.float32)
    Fv = (rng.standard_normal((kh, kw, shape[3], co)) * np.sqrt(2.0 / (kh * kw * shape[3]))).astype(np.float32)
    if kind == 'bf16':
        Iv, Fv = E.round_bf16(Iv), E.round_bf16(Fv)
    return Iv, Fv


# Shapes the resident-filter convolution takes (unit stride, 128 bytes of channels per pixel, CO <= 64):
# tiles of 256 pixels that run across image ends, odd widths, VALID and SAME windows, non-square filters.
RESIDENT_CASES = [('bf16', (3, 9, 30, 64), 3, 3, 64, op.SAME_UPPER), ('bf16', (2, 20, 40, 64), 3, 3, 40, op.VALID),
                  ('bf16', (2, 12, 33, 64), 2, 3, 48, op.VALID), ('bf16', (5, 17, 19, 64), 3, 3, 64, op.SAME_UPPER),
                  ('f32', (2, 12, 36, 32), 3, 3, 64, op.SAME_UPPER), ('i8', (2, 10, 30, 128), 3, 3, 64, op.SAME_UPPER)]


@pytest.mark.parametrize('kind,shape,kh,kw,co,autopad', RESIDENT_CASES)
def test_conv_resident_filter(kind, shape, kh, kw, co, autopad, capsys):
    Iv, Fv = _conv_case(kind, shape, kh, kw, co, autopad, 21)
    rng = np.random.default_rng(22)
    if kind == 'i8':
        out = run_conv(Iv, Fv, hk.I8, hk.I32, autopad=autopad)
        assert 'resident filter' in capsys.readouterr().out
        I, F = E.Placeholder(D.INT8, Iv.shape), E.Placeholder(D.INT8, Fv.shape)
        O = op.convolution(E.cast(I, D.INT32), E.cast(F, D.INT32), strides=[1, 1], autopad=autopad)
        ref, = E.run(E.Program('c', [I, F], [O]), [Iv, Fv])
        np.testing.assert_array_equal(out, ref)
        return
    bias = rng.standard_normal(co).astype(np.float32)
    if kind == 'bf16':
        bias = E.round_bf16(bias)
        out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, autopad=autopad, bias=bf16(bias), relu=True))
        ref = oracle_conv(Iv, Fv, D.BFLOAT16, 1, autopad, bias, True)
        np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2)
    else:
        out = run_conv(Iv, Fv, hk.F32, hk.F32, autopad=autopad, bias=bias, relu=True)
        ref = oracle_conv(Iv, Fv, D.FLOAT32, 1, autopad, bias, True)
        np.testing.assert_allclose(out, ref, rtol=FP32_RTOL, atol=1e-4)
    assert 'resident filter' in capsys.readouterr().out


# Windows of at most 10 rows of 32 to 64 pixels with 16- or 8-bit elements: the filter lives in registers.
# Ragged last tile, images that end inside a tile, the widest and the tallest window, VALID and SAME.
REGISTER_CASES = [('bf16', (2, 56, 56, 64), op.SAME_UPPER, True), ('bf16', (3, 11, 60, 64), op.SAME_UPPER, True),
                  ('bf16', (2, 9, 62, 64), op.VALID, False), ('bf16', (9, 9, 60, 64), op.SAME_UPPER, True),
                  ('i8', (2, 20, 50, 128), op.SAME_UPPER, False), ('i8', (1, 7, 47, 128), op.VALID, False)]


@pytest.mark.parametrize('kind,shape,autopad,with_bias', REGISTER_CASES)
def test_conv_register_filter(kind, shape, autopad, with_bias, capsys):
    Iv, Fv = _conv_case(kind, shape, 3, 3, 64, autopad, 27)
    if kind == 'i8':
        out = run_conv(Iv, Fv, hk.I8, hk.I32, autopad=autopad)
        assert 'in registers' in capsys.readouterr().out
        I, F = E.Placeholder(D.INT8, Iv.shape), E.Placeholder(D.INT8, Fv.shape)
        O = op.convolution(E.cast(I, D.INT32), E.cast(F, D.INT32), strides=[1, 1], autopad=autopad)
        ref, = E.run(E.Program('c', [I, F], [O]), [Iv, Fv])
        np.testing.assert_array_equal(out, ref)
        return
    bias = E.round_bf16(np.random.default_rng(28).standard_normal(64).astype(np.float32)) if with_bias else None
    out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, autopad=autopad,
                                    bias=bf16(bias) if with_bias else None, relu=with_bias))
    assert 'in registers' in capsys.readouterr().out
    ref = oracle_conv(Iv, Fv, D.BFLOAT16, 1, autopad, bias, with_bias)
    np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2)


@pytest.mark.parametrize('batch', [3, 24])
def test_conv_register_filter_matches_lds_filter(batch, monkeypatch):
    # same inputs with the filter kept in LDS: both accumulate in fp32 and round once.
    # batch 24 = 294 tiles on 256 workgroups: the 38 tiles of the last round are dealt out in halves
    Iv, Fv = _conv_case('bf16', (batch, 56, 56, 64), 3, 3, 64, op.SAME_UPPER, 29)
    bias = bf16(E.round_bf16(np.random.default_rng(30).standard_normal(64).astype(np.float32)))
    a = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True))
    monkeypatch.setitem(FORCED, 'flags', hk.flag_conv(hk.CONV_LDSFILTER))
    b = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True))
    np.testing.assert_allclose(a, b, rtol=BF16_RTOL, atol=1e-2)
    # the last image (part of the halved tiles when batch = 24) against a float64 evaluation of the definition
    Ip = np.pad(Iv[-1].astype(np.float64), ((1, 1), (1, 1), (0, 0)))
    ref = sum(np.einsum('yxc,cd->yxd', Ip[ky:ky + 56, kx:kx + 56], Fv[ky, kx].astype(np.float64))
              for ky in range(3) for kx in range(3))
    ref = np.maximum(ref + E.bf16_from_bits(bias).astype(np.float64), 0)
    np.testing.assert_allclose(a[-1], ref, rtol=BF16_RTOL, atol=2e-2)


@pytest.mark.parametrize('kind,shape', [('bf16', (5, 56, 56, 64)), ('bf16', (3, 20, 40, 64)), ('i8', (5, 56, 56, 128)),
                                        ('i8', (2, 30, 33, 128))])
def test_conv_filter_packed_once_equals_filter_per_call(kind, shape, capsys):
    """A constant 3x3 filter re-laid once (rows of 56 pixels: into the order the register-filter kernel holds it in
    registers; other shapes: as Bt, for whichever resident-filter kernel takes them) against the same filter handed over with every call, bit for bit; with a NaN, an
    infinity and a -0 product in the data, which relu must keep / keep / may store as +0."""
    rng = np.random.default_rng(61)
    if kind == 'bf16':
        Iv = E.round_bf16(rng.standard_normal(shape).astype(np.float32))
        Iv[0, 3, 3, 5], Iv[1, 0, 0, 0], Iv[2, 7, 9, :] = np.nan, np.inf, 0.0
        Fv = E.round_bf16((rng.standard_normal((3, 3, 64, 64)) * 0.06).astype(np.float32))
        bias = bf16(E.round_bf16(rng.standard_normal(64).astype(np.float32)))
        a = run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True)
        assert shape[2] != 56 or 'in registers' in capsys.readouterr().out
        b = run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True, packed=True)
        af = E.bf16_from_bits(a)
        assert np.isnan(af[0, 2:5, 2:5]).all() and np.isinf(af[1, 0, 0]).any()
    else:
        Iv = rng.integers(-127, 128, shape, dtype=np.int8)
        Fv = rng.integers(-127, 128, (3, 3, 128, 64), dtype=np.int8)
        a = run_conv(Iv, Fv, hk.I8, hk.I32, relu=True)
        assert shape[2] != 56 or 'in registers' in capsys.readouterr().out
        b = run_conv(Iv, Fv, hk.I8, hk.I32, relu=True, packed=True)
    np.testing.assert_array_equal(a, b)


def test_conv_resident_filter_general_tail(capsys):
    # relu(conv(I, F) + R) with a full-size residual R: the tail is interpreted, not the fast store path
    shape, co = (3, 9, 30, 64), 64
    Iv, Fv = _conv_case('bf16', shape, 3, 3, co, op.SAME_UPPER, 23)
    Rv = E.round_bf16(np.random.default_rng(24).standard_normal((3, 9, 30, co)).astype(np.float32))
    tail = hk.make_tail(ops=[(hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_RELU, hk.BF16, 0, 0, 0.0)],
                        operands=[(hk.BF16, co, 1)])
    out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, tail=tail, operands=[bf16(Rv)]))
    assert 'resident filter' in capsys.readouterr().out
    I, F, R = E.Placeholder(D.BFLOAT16, Iv.shape), E.Placeholder(D.BFLOAT16, Fv.shape), E.Placeholder(D.BFLOAT16, Rv.shape)
    O = op.relu(op.convolution(I, F, strides=[1, 1], autopad=op.SAME_UPPER) + R)
    ref, = E.run(E.Program('c', [I, F, R], [O]), [Iv, Fv, Rv])
    np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2)


def test_conv_resident_filter_matches_generic_kernel(monkeypatch):
    # same inputs through the generic implicit-GEMM kernel: both accumulate in fp32 and round once
    Iv, Fv = _conv_case('bf16', (4, 28, 28, 64), 3, 3, 64, op.SAME_UPPER, 25)
    bias = bf16(E.round_bf16(np.random.default_rng(26).standard_normal(64).astype(np.float32)))
    a = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True))
    monkeypatch.setitem(FORCED, 'flags', hk.flag_conv(hk.CONV_IGEMM))
    b = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, bias=bias, relu=True))
    np.testing.assert_allclose(a, b, rtol=BF16_RTOL, atol=1e-2)


def _stem_case(kind, shape, k, co, stride, pad, seed):
    Iv, Fv = _conv_case(kind, shape, k, k, co, op.SAME_UPPER, seed)
    bias = np.random.default_rng(seed + 1).standard_normal(co).astype(np.float32)
    if kind == 'bf16':
        bias = E.round_bf16(bias)
        out = E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, stride=stride, pad=pad, bias=bf16(bias),
                                        relu=True))
        ref = oracle_conv(Iv, Fv, D.BFLOAT16, stride, op.SAME_UPPER, bias, True, pad=pad)
        np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2)
    else:
        out = run_conv(Iv, Fv, hk.F32, hk.F32, stride=stride, pad=pad, bias=bias, relu=True,
                       flags=hk.FP32_AS_BF16X3 if kind == 'f32x3' else 0)
        ref = oracle_conv(Iv, Fv, D.FLOAT32, stride, op.SAME_UPPER, bias, True, pad=pad)
        np.testing.assert_allclose(out, ref, rtol=FP32_RTOL, atol=1e-4)


# stride 2 over channels that do not fill 16-byte vectors: unit-stride convolution over 2x2 pixel blocks.
# (shape, k, co, pad): even and odd padding, odd image sides, 1- and 5-channel images, a 3x3 and a 2x2 filter
STEM_CASES = [((2, 30, 34, 3), 7, 64, None), ((2, 32, 32, 3), 7, 64, 3), ((2, 31, 29, 3), 7, 64, 3),
              ((3, 17, 23, 1), 3, 32, 1), ((1, 20, 18, 5), 5, 48, 0), ((2, 16, 16, 3), 2, 64, 0),
              # many images (a workgroup of the row-walking bf16 kernel takes several output rows, the last run ragged)
              # and a wide one (four 32-pixel blocks per row, the last ragged)
              ((40, 30, 34, 3), 7, 64, None), ((1, 64, 200, 3), 7, 64, 3),
              # an odd height with an even width: the kernel builds the pixel blocks itself and the last block row
              # has no second image row
              ((2, 31, 30, 3), 7, 64, 3), ((1, 9, 8, 3), 7, 64, None)]


@pytest.mark.parametrize('kind', ['f32', 'bf16', 'f32x3'])
@pytest.mark.parametrize('shape,k,co,pad', STEM_CASES)
def test_conv_few_channel_stride2(kind, shape, k, co, pad, capsys):
    _stem_case(kind, shape, k, co, 2, pad, 41)
    text = capsys.readouterr().out
    assert '2x2 pixel blocks' in text
    # 7x7 (4x4 block taps) onto 64 channels in bf16 is the row-walking kernel's case: no silent fall-back to the implicit GEMM
    if kind == 'bf16' and k == 7 and co == 64:
        assert 'row by row with the filter in registers' in text


# Runs of two and more output rows per workgroup take the row-walking kernel's eight-wavefront form (a pixel's 128
# bytes then come from two wavefronts, through LDS, one row late): ragged last runs, a second pixel block that is half
# empty with two idle wavefront pairs, four pixel blocks with a ragged last one.  The first case against the oracle;
# the larger ones, which the oracle would take minutes over, against the implicit-GEMM path of the same library
# (itself held to the oracle by the cases above).
@pytest.mark.parametrize('shape,pad,against_oracle', [((256, 14, 34, 3), None, True), ((96, 62, 70, 3), 3, False),
                                                      ((128, 26, 250, 3), 3, False)])
def test_conv_stem_long_runs(shape, pad, against_oracle, capsys):
    if against_oracle:
        _stem_case('bf16', shape, 7, 64, 2, pad, 47)
        assert 'row by row with the filter in registers' in capsys.readouterr().out
        return
    Iv, Fv = _conv_case('bf16', shape, 7, 7, 64, op.SAME_UPPER, 47)
    bias = E.round_bf16(np.random.default_rng(48).standard_normal(64).astype(np.float32))
    outs = []
    for flags in (0, hk.flag_conv(hk.CONV_IGEMM)):
        outs.append(E.bf16_from_bits(run_conv(bf16(Iv), bf16(Fv), hk.BF16, hk.BF16, stride=2, pad=pad, bias=bf16(bias), relu=True,
                                              flags=flags)))
    text = capsys.readouterr().out
    assert text.count('row by row with the filter in registers') == 1
    np.testing.assert_allclose(outs[0], outs[1], rtol=BF16_RTOL, atol=1e-2)


# The stem convolution with its 3x3 stride-2 max-pool inside the launch (PML_HIP_FLAG_MAXPOOL3x3S2) against the same
# convolution followed by pml_hip_pool2d, bit for bit.  (shape, conv pad, pool pads top / bottom / left / right): the
# network shape in small (SAME_UPPER pooling of an even side: one row and column of padding behind), padding in front,
# on both sides and none, odd sides, a last window cut off by the image's end, rows of more than one pixel block with a
# ragged last block, many images (several pooled rows per workgroup) and one (a pooled row per workgroup)
MAXPOOL_CASES = [((8, 64, 64, 3), 3, (0, 1, 0, 1)), ((3, 30, 34, 3), None, (1, 1, 1, 1)), ((2, 31, 29, 3), 3, (1, 0, 1, 0)),
                 ((5, 40, 140, 3), 3, (0, 0, 0, 0)), ((160, 24, 70, 3), 3, (0, 1, 1, 1)), ((1, 64, 200, 3), 3, (0, 1, 0, 1)),
                 ((2, 14, 16, 3), 3, (1, 1, 0, 0))]


@pytest.mark.parametrize('shape,pad,pp', MAXPOOL_CASES)
def test_conv_stem_with_maxpool_inside(shape, pad, pp):
    L = hk.lib()
    Iv, Fv = _conv_case('bf16', shape, 7, 7, 64, op.SAME_UPPER, 51)
    bias = bf16(E.round_bf16(np.random.default_rng(52).standard_normal(64).astype(np.float32)))
    N, H, W, CI = shape
    # infinities of both signs in the image: convolution results that are +infinity, and NaN (which no window may pick;
    # a window of nothing but NaN pools to -infinity)
    Iv = Iv.copy()
    Iv[0, H // 2, W // 2, :] = np.inf
    Iv[0, H // 2 + 1, W // 2 + 1, 0] = -np.inf
    Iv[N - 1, 2:12, 2:12, 1] = np.inf
    Iv[N - 1, 3:11, 3:11, 2] = -np.inf
    ph, OH = op.compute_padding_and_output_size(H, 7, 2, op.SAME_UPPER)
    pw, OW = op.compute_padding_and_output_size(W, 7, 2, op.SAME_UPPER)
    if pad is not None:
        ph = pw = pad
        OH, OW = (H + 2 * pad - 7) // 2 + 1, (W + 2 * pad - 7) // 2 + 1
    pt, pb, pl, pr = pp
    POH, POW = (OH + pt + pb - 3) // 2 + 1, (OW + pl + pr - 3) // 2 + 1

    def conv_desc(flags):
        d = hk.Conv2dDesc()
        d.in_dtype = d.out_dtype = d.c_dtype = hk.BF16
        d.flags = flags
        d.n, d.h, d.w, d.ci, d.kh, d.kw, d.co, d.oh, d.ow = N, H, W, CI, 7, 7, 64, OH, OW
        d.stride_h = d.stride_w = 2
        d.dil_h = d.dil_w = 1
        d.pad_h, d.pad_w = ph, pw
        d.init_kind, d.init_dtype = 1, hk.BF16
        d.init_row_stride, d.init_col_stride = 0, 1
        d.tail = hk.make_tail(ops=[(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)])
        return d
    dI, dF, dB = hk.DeviceBuffer.from_numpy(bf16(Iv)), hk.DeviceBuffer.from_numpy(bf16(Fv)), hk.DeviceBuffer.from_numpy(bias)
    none = hk.ptr_array([])
    # the two launches
    d = conv_desc(0)
    plan = L.pml_hip_conv2d_dispatch(ctypes.byref(d))
    assert plan, L.pml_hip_last_error()
    dC = hk.DeviceBuffer(N * OH * OW * 64 * 2)
    hk.check(L.pml_hip_conv2d_invoke(plan, dI.ptr, dF.ptr, dC.ptr, dB.ptr, none, none, None))
    q = hk.Pool2dDesc()
    q.dtype, q.agg = hk.BF16, hk.AGG_MAX
    q.n, q.h, q.w, q.c, q.kh, q.kw, q.oh, q.ow = N, OH, OW, 64, 3, 3, POH, POW
    q.stride_h = q.stride_w = 2
    q.pad_h, q.pad_w = pt, pl
    plan2 = L.pml_hip_pool2d_dispatch(ctypes.byref(q))
    assert plan2, L.pml_hip_last_error()
    dP = hk.DeviceBuffer(N * POH * POW * 64 * 2)
    hk.check(L.pml_hip_pool2d_invoke(plan2, dC.ptr, dP.ptr, None, None))
    hk.check(L.pml_hip_stream_sync(None))
    apart = dP.to_numpy(np.uint16, (N, POH, POW, 64))
    # one launch
    f = conv_desc(hk.flag_maxpool3x3s2(pt, pb, pl, pr))
    assert L.pml_hip_conv2d_takes_maxpool(ctypes.byref(f)) == 1
    plan3 = L.pml_hip_conv2d_dispatch(ctypes.byref(f))
    assert plan3, L.pml_hip_last_error()
    assert 'max-pool 3x3 stride 2 -> %dx%d' % (POH, POW) in hk.describe(plan3)
    dQ = hk.DeviceBuffer(N * POH * POW * 64 * 2)
    dQ.fill_u32(0x7fc07fc0)
    hk.check(L.pml_hip_conv2d_invoke(plan3, dI.ptr, dF.ptr, dQ.ptr, dB.ptr, none, none, None))
    hk.check(L.pml_hip_stream_sync(None))
    fused = dQ.to_numpy(np.uint16, (N, POH, POW, 64))
    np.testing.assert_array_equal(fused, apart)
    assert not np.isnan(E.bf16_from_bits(fused)).any()
    for pl_ in (plan, plan2, plan3):
        L.pml_hip_plan_free(pl_)


def test_conv_maxpool_inside_is_refused_elsewhere():
    """Only the row-walking stem kernel has the pool: other convolutions refuse the flag at dispatch, and say so."""
    L = hk.lib()
    d = hk.Conv2dDesc()
    d.in_dtype = d.out_dtype = d.c_dtype = hk.BF16
    d.flags = hk.flag_maxpool3x3s2(0, 1, 0, 1)
    d.n, d.h, d.w, d.ci, d.kh, d.kw, d.co, d.oh, d.ow = 2, 16, 16, 64, 3, 3, 64, 16, 16
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.pad_h = d.pad_w = 1
    assert L.pml_hip_conv2d_takes_maxpool(ctypes.byref(d)) == 0
    assert L.pml_hip_conv2d_dispatch(ctypes.byref(d)) == 0
    assert 'fused max-pool' in L.pml_hip_last_error().decode()


@pytest.mark.parametrize('kind', ['f32', 'bf16', 'f32x3'])
@pytest.mark.parametrize('stride', [1, 2])
def test_conv_few_channel_patch_matrix(kind, stride, capsys, monkeypatch):
    # other strides (and stride 2 on request) gather a patch matrix [M][K padded] and run a plain GEMM
    monkeypatch.setitem(FORCED, 'flags', hk.flag_conv(hk.CONV_PATCHES))
    _stem_case(kind, (2, 30, 34, 3), 7, 64, stride, None, 43)
    assert 'patch matrix' in capsys.readouterr().out


# (dtype, N, H, W, C, k, stride, pad): the 3x3 unit-stride kernel that computes four pixels per thread (widths
# that are and are not multiples of four, SAME and VALID windows, an infinity in the filter that a padded tap
# must not turn into NaN) and the general one (5x5, stride 2)
DW_CASES = [('bf16', 2, 19, 19, 32, 3, 1, 1), ('bf16', 1, 9, 24, 16, 3, 1, 0), ('f32', 2, 11, 13, 8, 3, 1, 1),
            ('bf16', 1, 12, 15, 16, 5, 1, 2), ('f32', 1, 14, 14, 8, 3, 2, 1)]


@pytest.mark.parametrize('packed', [False, True, 'finite'])
@pytest.mark.parametrize('kind,N,H,W,C,k,stride,pad', DW_CASES)
def test_dwconv_shapes(kind, N, H, W, C, k, stride, pad, packed):
    """packed: the filter is handed over once (pml_hip_dwconv2d_pack_filter) and the invoke is given none -- with the
    infinite weight, which keeps the general kernel, and ('finite') without it, which lets the 3x3 bf16 case take the
    kernel that multiplies the taps of two filter rows in one instruction."""
    rng = np.random.default_rng(90)
    Iv = rng.standard_normal((N, H, W, C)).astype(np.float32)
    Fv = (rng.standard_normal((k, k, C, 1)) * 0.3).astype(np.float32)
    with_inf = k == 3 and stride == 1 and pad == 1 and packed != 'finite'
    if with_inf:
        Fv[0, 0, 0, 0] = np.inf  # only pixels whose top-left tap lies inside the image see it
    if kind == 'bf16':
        Iv, Fv = E.round_bf16(Iv), E.round_bf16(Fv)
    OH, OW = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    d = hk.Dwconv2dDesc()
    d.dtype = hk.BF16 if kind == 'bf16' else hk.F32
    d.n, d.h, d.w, d.c, d.kh, d.kw, d.oh, d.ow = N, H, W, C, k, k, OH, OW
    d.stride_h = d.stride_w = stride
    d.dil_h = d.dil_w = 1
    d.pad_h = d.pad_w = pad
    plan = hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d))
    assert plan, hk.lib().pml_hip_last_error()
    es = 2 if kind == 'bf16' else 4
    dI = hk.DeviceBuffer.from_numpy(bf16(Iv) if kind == 'bf16' else Iv)
    dF = hk.DeviceBuffer.from_numpy(bf16(Fv) if kind == 'bf16' else Fv)
    dO = hk.DeviceBuffer(N * OH * OW * C * es)
    if packed:
        hk.check(hk.lib().pml_hip_dwconv2d_pack_filter(plan, dF.ptr, None))
        hk.check(hk.lib().pml_hip_fill_u32(dF.ptr, 0x7fc07fc0, k * k * C * es // 4, None))  # the plan keeps its own copy
    hk.check(hk.lib().pml_hip_dwconv2d_invoke(plan, dI.ptr, None if packed else dF.ptr, dO.ptr, hk.ptr_array([]), hk.ptr_array([]), None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    out = dO.to_numpy(np.uint16 if kind == 'bf16' else np.float32, (N, OH, OW, C))
    if kind == 'bf16':
        out = E.bf16_from_bits(out)
    dt = D.BFLOAT16 if kind == 'bf16' else D.FLOAT32
    I, F = E.Placeholder(dt, Iv.shape), E.Placeholder(dt, Fv.shape)
    O = op.convolution(I, F, strides=[stride, stride], autopad=op.EXPLICIT, manual_padding=[pad, pad], depthwise=True)
    ref, = E.run(E.Program('dw', [I, F], [O]), [Iv, Fv])
    assert np.isinf(ref).any() == with_inf and not np.isnan(ref).any()
    np.testing.assert_allclose(out, ref, rtol=BF16_RTOL if kind == 'bf16' else FP32_RTOL, atol=1e-2 if kind == 'bf16' else 1e-4)
    hk.lib().pml_hip_plan_free(plan)


# (dtype, N, H, W, C, pad, with an infinite weight): 3x3 unit-stride cases with enough threads for the kernel that walks
# down the image with the window rows in registers -- runs of rows with a ragged last one, an odd width (the last
# pixel pair is half empty), SAME, VALID and a wider padding, lanes with an infinite weight next to lanes without
DW_WALK_CASES = [('bf16', 16, 19, 19, 728, 1, True), ('bf16', 16, 19, 19, 728, 1, False), ('bf16', 64, 12, 40, 256, 0, False),
                 ('f32', 24, 20, 21, 512, 2, True), ('f32', 12, 33, 18, 512, 1, False),
                 # images of two rows and of one: runs shorter than the three rows a window spans
                 ('bf16', 2048, 2, 3, 256, 1, False), ('f32', 4096, 1, 5, 64, 1, True)]


@pytest.mark.parametrize('packed', [False, True])
@pytest.mark.parametrize('kind,N,H,W,C,pad,with_inf', DW_WALK_CASES)
def test_dwconv_rows_walked_in_registers(kind, N, H, W, C, pad, with_inf, packed):
    rng = np.random.default_rng(92)
    Iv = rng.standard_normal((N, H, W, C)).astype(np.float32)
    Fv = (rng.standard_normal((3, 3, C, 1)) * 0.3).astype(np.float32)
    if with_inf:
        Fv[0, 0, 0, 0] = np.inf   # a corner tap: padded for the first row and column only
        Fv[2, 1, C - 1, 0] = -np.inf
    if kind == 'bf16':
        Iv, Fv = E.round_bf16(Iv), E.round_bf16(Fv)
    OH, OW = H + 2 * pad - 2, W + 2 * pad - 2
    es = 2 if kind == 'bf16' else 4
    outs = []
    for pitch in (0, C + 2 * (16 // es)):
        d = hk.Dwconv2dDesc()
        d.dtype = hk.BF16 if kind == 'bf16' else hk.F32
        d.out_pitch = pitch
        d.n, d.h, d.w, d.c, d.kh, d.kw, d.oh, d.ow = N, H, W, C, 3, 3, OH, OW
        d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
        d.pad_h = d.pad_w = pad
        plan = hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d))
        assert plan, hk.lib().pml_hip_last_error()
        assert 'window rows walked in registers' in hk.describe(plan)
        dI = hk.DeviceBuffer.from_numpy(bf16(Iv) if kind == 'bf16' else Iv)
        dF = hk.DeviceBuffer.from_numpy(bf16(Fv) if kind == 'bf16' else Fv)
        width = pitch or C
        dO = hk.DeviceBuffer(N * OH * OW * width * es)
        dO.fill_u32(0x12341234)
        if packed:
            hk.check(hk.lib().pml_hip_dwconv2d_pack_filter(plan, dF.ptr, None))
        hk.check(hk.lib().pml_hip_dwconv2d_invoke(plan, dI.ptr, None if packed else dF.ptr, dO.ptr, hk.ptr_array([]), hk.ptr_array([]), None))
        hk.check(hk.lib().pml_hip_stream_sync(None))
        outs.append(dO.to_numpy(np.uint16 if es == 2 else np.uint32, (N * OH * OW, width)))
        hk.lib().pml_hip_plan_free(plan)
    dense, pitched = outs
    # the pitched result: the same bits, the bytes between a pixel's channels and the next pixel left alone
    np.testing.assert_array_equal(pitched[:, :C], dense)
    assert (pitched[:, C:] == (0x1234 if es == 2 else 0x12341234)).all()
    out = E.bf16_from_bits(dense.reshape(N, OH, OW, C)) if es == 2 else dense.view(np.float32).reshape(N, OH, OW, C)
    dt = D.BFLOAT16 if kind == 'bf16' else D.FLOAT32
    I, F = E.Placeholder(dt, Iv.shape), E.Placeholder(dt, Fv.shape)
    O = op.convolution(I, F, strides=[1, 1], autopad=op.EXPLICIT, manual_padding=[pad, pad], depthwise=True)
    ref, = E.run(E.Program('dw', [I, F], [O]), [Iv, Fv])
    # (in an image of one row both infinite weights only ever meet taps outside it: nothing infinite, and no NaN)
    assert np.isinf(ref).any() == (with_inf and H > 1) and not np.isnan(ref).any()
    np.testing.assert_allclose(out, ref, rtol=BF16_RTOL if kind == 'bf16' else FP32_RTOL, atol=1e-2 if kind == 'bf16' else 1e-4)


@pytest.mark.parametrize('kind,N,H,W,C,k,stride,pad', DW_CASES[:3] + DW_CASES[4:])
def test_dwconv_output_pitch(kind, N, H, W, C, k, stride, pad):
    """With an output pitch the same values land `pitch` elements apart, bit for bit, and the bytes between a
    pixel's channels and the next pixel are left alone; a pitch that is no whole number of 16-byte vectors, or
    smaller than c, or combined with a tail, is refused."""
    rng = np.random.default_rng(91)
    es, npdt = (2, np.uint16) if kind == 'bf16' else (4, np.float32)
    Iv = rng.standard_normal((N, H, W, C)).astype(np.float32)
    Fv = (rng.standard_normal((k, k, C, 1)) * 0.3).astype(np.float32)
    OH, OW = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    pitch = C + 3 * (16 // es)
    outs = []
    for op_pitch in (0, pitch):
        d = hk.Dwconv2dDesc()
        d.dtype = hk.BF16 if kind == 'bf16' else hk.F32
        d.out_pitch = op_pitch
        d.n, d.h, d.w, d.c, d.kh, d.kw, d.oh, d.ow = N, H, W, C, k, k, OH, OW
        d.stride_h = d.stride_w = stride
        d.dil_h = d.dil_w = 1
        d.pad_h = d.pad_w = pad
        plan = hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d))
        assert plan, hk.lib().pml_hip_last_error()
        dI = hk.DeviceBuffer.from_numpy(bf16(Iv) if kind == 'bf16' else Iv)
        dF = hk.DeviceBuffer.from_numpy(bf16(Fv) if kind == 'bf16' else Fv)
        width = op_pitch or C
        dO = hk.DeviceBuffer.from_numpy(np.full((N * OH * OW, width), 0x1234 if kind == 'bf16' else 7.5, npdt))
        hk.check(hk.lib().pml_hip_dwconv2d_invoke(plan, dI.ptr, dF.ptr, dO.ptr, hk.ptr_array([]), hk.ptr_array([]), None))
        hk.check(hk.lib().pml_hip_stream_sync(None))
        outs.append(dO.to_numpy(npdt, (N * OH * OW, width)))
        hk.lib().pml_hip_plan_free(plan)
    dense, pitched = outs
    np.testing.assert_array_equal(pitched[:, :C].view(np.uint16 if es == 2 else np.uint32), dense.view(np.uint16 if es == 2 else np.uint32))
    assert (pitched[:, C:] == (0x1234 if kind == 'bf16' else 7.5)).all()
    for bad in (C - 16 // es, C + 1):
        d.out_pitch = bad
        assert hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d)) == 0
        assert 'output pitch' in hk.lib().pml_hip_last_error().decode()
    d.out_pitch = pitch
    d.tail = hk.make_tail(ops=[(hk.EPI_RELU, d.dtype, 0, 0, 0.0)], operands=[])
    assert hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d)) == 0


def test_dwconv_pool_bf16():
    rng = np.random.default_rng(9)
    N, H, W, C = 2, 19, 19, 32
    Iv = E.round_bf16(rng.standard_normal((N, H, W, C)).astype(np.float32))
    Fv = E.round_bf16((rng.standard_normal((3, 3, C, 1)) * 0.3).astype(np.float32))
    d = hk.Dwconv2dDesc()
    d.dtype = hk.BF16
    d.n, d.h, d.w, d.c, d.kh, d.kw, d.oh, d.ow = N, H, W, C, 3, 3, H, W
    d.stride_h = d.stride_w = d.dil_h = d.dil_w = 1
    d.pad_h = d.pad_w = 1
    plan = hk.lib().pml_hip_dwconv2d_dispatch(ctypes.byref(d))
    assert plan, hk.lib().pml_hip_last_error()
    dI, dF = hk.DeviceBuffer.from_numpy(bf16(Iv)), hk.DeviceBuffer.from_numpy(bf16(Fv))
    dO = hk.DeviceBuffer(N * H * W * C * 2)
    hk.check(hk.lib().pml_hip_dwconv2d_invoke(plan, dI.ptr, dF.ptr, dO.ptr, hk.ptr_array([]), hk.ptr_array([]), None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    out = E.bf16_from_bits(dO.to_numpy(np.uint16, (N, H, W, C)))
    I, F = E.Placeholder(D.BFLOAT16, Iv.shape), E.Placeholder(D.BFLOAT16, Fv.shape)
    ref, = E.run(E.Program('dw', [I, F], [op.convolution(I, F, depthwise=True)]), [Iv, Fv])
    np.testing.assert_allclose(out, ref, rtol=BF16_RTOL, atol=1e-2)

    # max-pool 3x3/2 SAME with window argmax; ties forced by quantising the input
    Pv = E.round_bf16(np.round(Iv * 2) / 2)
    p = hk.Pool2dDesc()
    p.dtype, p.agg = hk.BF16, hk.AGG_MAX
    p.n, p.h, p.w, p.c, p.kh, p.kw, p.oh, p.ow = N, H, W, C, 3, 3, 10, 10
    p.stride_h = p.stride_w = 2
    p.pad_h = p.pad_w = 1
    p.with_index = 1
    plan2 = hk.lib().pml_hip_pool2d_dispatch(ctypes.byref(p))
    assert plan2, hk.lib().pml_hip_last_error()
    dP = hk.DeviceBuffer.from_numpy(bf16(Pv))
    dM, dX = hk.DeviceBuffer(N * 10 * 10 * C * 2), hk.DeviceBuffer(N * 10 * 10 * C * 4)
    hk.check(hk.lib().pml_hip_pool2d_invoke(plan2, dP.ptr, dM.ptr, dX.ptr, None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    m = E.bf16_from_bits(dM.to_numpy(np.uint16, (N, 10, 10, C)))
    ix = dX.to_numpy(np.int32, (N, 10, 10, C))
    R = E.Placeholder(D.BFLOAT16, Pv.shape)
    M = op.pool(R, 'max', [3, 3], [2, 2], autopad=op.SAME_UPPER)
    n_, x0, x1, c, k0, k1 = E.TensorIndexes(6)
    IX = E.index([3, 3], 0) * 3 + E.index([3, 3], 1)
    AM = E.Contraction().outShape(M.shape).outAccess(n_, x0, x1, c).max(
        E.cond(R[n_, 2 * x0 + k0 - 1, 2 * x1 + k1 - 1, c], M[n_, x0, x1, c], IX[k0, k1])).build()
    mo, ao = E.run(E.Program('pool', [R], [M, AM]), [Pv])
    np.testing.assert_array_equal(m, mo)
    np.testing.assert_array_equal(ix, ao)
    hk.lib().pml_hip_plan_free(plan)
    hk.lib().pml_hip_plan_free(plan2)


@pytest.mark.gpu
@pytest.mark.parametrize('kind,agg,N,H,W,C,divisor', [
    ('bf16', 'add', 3, 7, 7, 2048, 0), ('bf16', 'max', 2, 7, 7, 264, 0), ('bf16', 'min', 2, 10, 13, 64, 0),
    ('f32', 'add', 2, 7, 7, 516, 0), ('f32', 'max', 1, 9, 8, 128, 0), ('f32', 'add', 2, 4, 4, 36, 0), ('bf16', 'add', 2, 3, 3, 64, 0),
    ('bf16', 'add', 3, 7, 7, 2048, 49), ('f32', 'add', 2, 7, 7, 516, 49), ('bf16', 'add', 1, 5, 4, 72, 20)])
def test_pool_whole_image(kind, agg, N, H, W, C, divisor):
    """Pooling over the whole image (taps shared by eight threads when there are at least 16; the plain window
    kernel below that) against numpy: max / min exactly, sums to the accumulation tolerance.  With a divisor (a mean
    as sum / count in one launch) the sum is rounded to the element type before the division, as two launches would."""
    print('whole-image pool', kind, agg, N, H, W, C, divisor, flush=True)
    rng = np.random.default_rng(N * 1000 + C)
    Iv = rng.standard_normal((N, H, W, C)).astype(np.float32)
    if kind == 'bf16':
        Iv = E.round_bf16(Iv)
    p = hk.Pool2dDesc()
    p.dtype = hk.BF16 if kind == 'bf16' else hk.F32
    p.agg = {'add': hk.AGG_ADD, 'max': hk.AGG_MAX, 'min': hk.AGG_MIN}[agg]
    p.n, p.h, p.w, p.c, p.kh, p.kw, p.oh, p.ow = N, H, W, C, H, W, 1, 1
    p.stride_h = p.stride_w = 1
    p.divisor = divisor
    plan = hk.lib().pml_hip_pool2d_dispatch(ctypes.byref(p))
    assert plan, hk.lib().pml_hip_last_error()
    es = 2 if kind == 'bf16' else 4
    dI = hk.DeviceBuffer.from_numpy(bf16(Iv) if kind == 'bf16' else Iv)
    dO = hk.DeviceBuffer(N * C * es)
    hk.check(hk.lib().pml_hip_pool2d_invoke(plan, dI.ptr, dO.ptr, None, None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    out = E.bf16_from_bits(dO.to_numpy(np.uint16, (N, C))) if kind == 'bf16' else dO.to_numpy(np.float32, (N, C))
    flat = Iv.reshape(N, H * W, C)
    if agg == 'add' and divisor:
        # the two-launch form on the same device: sum, then the division as an elementwise launch of its own
        p.divisor = 0
        plan0 = hk.lib().pml_hip_pool2d_dispatch(ctypes.byref(p))
        dS = hk.DeviceBuffer(N * C * es)
        hk.check(hk.lib().pml_hip_pool2d_invoke(plan0, dI.ptr, dS.ptr, None, None))
        hk.check(hk.lib().pml_hip_stream_sync(None))
        sums = E.bf16_from_bits(dS.to_numpy(np.uint16, (N, C))) if kind == 'bf16' else dS.to_numpy(np.float32, (N, C))
        apart = (sums.astype(np.float32) / np.float32(divisor)).astype(np.float32)
        np.testing.assert_array_equal(out, E.round_bf16(apart) if kind == 'bf16' else apart)
        np.testing.assert_allclose(out, flat.astype(np.float64).sum(1) / divisor, rtol=BF16_RTOL if kind == 'bf16' else 1e-5,
                                   atol=2e-2 if kind == 'bf16' else 1e-5)
        hk.lib().pml_hip_plan_free(plan0)
    elif agg == 'add':
        ref = flat.astype(np.float64).sum(1)
        np.testing.assert_allclose(out, ref, rtol=BF16_RTOL if kind == 'bf16' else 1e-5, atol=2e-2 if kind == 'bf16' else 1e-5)
    else:
        np.testing.assert_array_equal(out, flat.max(1) if agg == 'max' else flat.min(1))
    hk.lib().pml_hip_plan_free(plan)


@pytest.mark.gpu
@pytest.mark.parametrize('kind,rows,cols', [('bf16', 1, 1000), ('bf16', 128, 1000), ('f32', 3, 5), ('f32', 2, 4097), ('bf16', 5, 257)])
def test_softmax_rows(kind, rows, cols):
    """pml_hip_softmax against the five operations it stands for, evaluated in numpy with the roundings they would make
    (bf16: after the subtraction, the exponential, the sum and the quotient).  The fp32 sum is accumulated in another
    order than numpy's, so sums and quotients are compared to a few units in the last place of the result type."""
    print('softmax', kind, rows, cols, flush=True)
    rng = np.random.default_rng(rows * 31 + cols)
    X = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    rnd = E.round_bf16 if kind == 'bf16' else (lambda a: a.astype(np.float32))
    X = rnd(X)
    d = hk.SoftmaxDesc()
    d.dtype, d.rows, d.cols = (hk.BF16 if kind == 'bf16' else hk.F32), rows, cols
    dX = hk.DeviceBuffer.from_numpy(bf16(X) if kind == 'bf16' else X)
    dY = hk.DeviceBuffer(rows * cols * (2 if kind == 'bf16' else 4))
    hk.check(hk.lib().pml_hip_softmax(ctypes.byref(d), dX.ptr, dY.ptr, None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    Y = E.bf16_from_bits(dY.to_numpy(np.uint16, (rows, cols))) if kind == 'bf16' else dY.to_numpy(np.float32, (rows, cols))
    m = X.max(axis=1, keepdims=True)
    e = rnd(np.exp(rnd(X - m).astype(np.float64)).astype(np.float32))
    ssum = rnd(e.astype(np.float64).sum(axis=1, keepdims=True).astype(np.float32))
    ref = rnd((e / ssum).astype(np.float32))
    tol = 2.0 ** -7 if kind == 'bf16' else 1e-5   # one bf16 step of the sum moves every quotient of its row by one step
    np.testing.assert_allclose(Y, ref, rtol=tol, atol=1e-30)
    np.testing.assert_allclose(Y.astype(np.float64).sum(axis=1), 1.0, rtol=0, atol=2e-2 if kind == 'bf16' else 1e-5)


# (kind, agg, N, H, W, C, kh, kw, stride, pad, with_index): the straight-line kernels (3x3, 2x2) and the window loop
# (5x5, 3x2), windows that cross every border, one image and several, values quantised so that ties occur
POOL_WINDOW_CASES = [
    ('bf16', 'max', 2, 19, 19, 24, 3, 3, 2, 1, 1), ('bf16', 'max', 1, 8, 11, 16, 2, 2, 2, 0, 1), ('f32', 'max', 2, 9, 7, 8, 3, 3, 1, 1, 1),
    ('bf16', 'min', 2, 10, 10, 16, 3, 3, 2, 1, 1), ('f32', 'min', 1, 6, 6, 12, 2, 2, 1, 0, 0), ('bf16', 'add', 2, 12, 9, 16, 3, 3, 2, 1, 0),
    ('f32', 'add', 3, 7, 7, 4, 2, 2, 2, 1, 0), ('bf16', 'max', 2, 14, 14, 8, 5, 5, 2, 2, 1), ('f32', 'max', 1, 9, 9, 4, 3, 2, 1, 1, 0),
    ('bf16', 'max', 1, 112, 112, 64, 3, 3, 2, 1, 0)]


@pytest.mark.gpu
@pytest.mark.parametrize('kind,agg,N,H,W,C,kh,kw,stride,pad,with_index', POOL_WINDOW_CASES)
def test_pool_windows_against_enumeration(kind, agg, N, H, W, C, kh, kw, stride, pad, with_index):
    """Every output against a direct enumeration of its window: taps outside the image take no part; the index output
    is the largest tap number kh_i * KW + kw_i whose value equals the pooled one (bit-exact, ties included)."""
    print('pool window', kind, agg, N, H, W, C, kh, kw, stride, pad, with_index, flush=True)
    rng = np.random.default_rng(H * 100 + W + C)
    Iv = (np.round(rng.standard_normal((N, H, W, C)) * 4) / 4).astype(np.float32)
    OH, OW = (H + 2 * pad - kh) // stride + 1, (W + 2 * pad - kw) // stride + 1
    p = hk.Pool2dDesc()
    p.dtype = hk.BF16 if kind == 'bf16' else hk.F32
    p.agg = {'add': hk.AGG_ADD, 'max': hk.AGG_MAX, 'min': hk.AGG_MIN}[agg]
    p.n, p.h, p.w, p.c, p.kh, p.kw, p.oh, p.ow = N, H, W, C, kh, kw, OH, OW
    p.stride_h = p.stride_w = stride
    p.pad_h = p.pad_w = pad
    p.with_index = with_index
    plan = hk.lib().pml_hip_pool2d_dispatch(ctypes.byref(p))
    assert plan, hk.lib().pml_hip_last_error()
    es = 2 if kind == 'bf16' else 4
    dI = hk.DeviceBuffer.from_numpy(bf16(Iv) if kind == 'bf16' else Iv)
    dO = hk.DeviceBuffer(N * OH * OW * C * es)
    dX = hk.DeviceBuffer(N * OH * OW * C * 4) if with_index else None
    hk.check(hk.lib().pml_hip_pool2d_invoke(plan, dI.ptr, dO.ptr, dX.ptr if dX else None, None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    out = E.bf16_from_bits(dO.to_numpy(np.uint16, (N, OH, OW, C))) if kind == 'bf16' else dO.to_numpy(np.float32, (N, OH, OW, C))
    ident = {'add': 0.0, 'max': -np.inf, 'min': np.inf}[agg]
    ref = np.full((N, OH, OW, C), ident, np.float64)
    best = np.zeros((N, OH, OW, C), np.int32)
    taps = []
    for ky in range(kh):
        for kx in range(kw):
            tap = np.full((N, OH, OW, C), np.nan)
            for oy in range(OH):
                iy = oy * stride + ky - pad
                if not 0 <= iy < H:
                    continue
                for ox in range(OW):
                    ix = ox * stride + kx - pad
                    if 0 <= ix < W:
                        tap[:, oy, ox] = Iv[:, iy, ix]
            taps.append(tap)
            live = ~np.isnan(tap)
            if agg == 'add':
                ref = np.where(live, ref + np.nan_to_num(tap), ref)
            elif agg == 'max':
                ref = np.where(live & (tap > ref), tap, ref)
            else:
                ref = np.where(live & (tap < ref), tap, ref)
    for k, tap in enumerate(taps):
        best = np.where(tap == ref, np.int32(k), best)  # NaN (outside) never equals
    if agg == 'add':
        np.testing.assert_allclose(out, ref, rtol=BF16_RTOL if kind == 'bf16' else 1e-6, atol=1e-6)
    else:
        np.testing.assert_array_equal(out, ref.astype(np.float32))
    if with_index:
        np.testing.assert_array_equal(dX.to_numpy(np.int32, (N, OH, OW, C)), best)
    hk.lib().pml_hip_plan_free(plan)


# (M, N, K): many rows, whole 128-column tiles, K of one slab, of three with a 16-byte tail, of four
def _gemm_f32_layouts(A, B_kn, ldb, flags, packed_first=False):
    """A . B for an fp32 right-hand side handed over as [K][N] at leading dimension ldb, and for the same values as
    [N][K] (K contiguous): both results."""
    M, K = A.shape
    N = B_kn.shape[1]
    out = []
    for layout in (0, 1):
        d = hk.GemmDesc()
        d.in_dtype = d.out_dtype = d.c_dtype = hk.F32
        d.flags = flags | FORCED['flags']
        d.m, d.n, d.k = M, N, K
        d.lda, d.ldc = K, N
        d.b_layout = layout
        if layout == 0:
            Bh = np.zeros((K, ldb), np.float32)
            Bh[:, :N] = B_kn
            Bh[:, N:] = np.nan  # what lies between the rows must never be read into a product
            d.ldb = ldb
        else:
            Bh = np.ascontiguousarray(B_kn.T)
            d.ldb = K
        plan = hk.lib().pml_hip_gemm_dispatch(ctypes.byref(d))
        assert plan, hk.lib().pml_hip_last_error()
        dA, dB, dC = hk.DeviceBuffer.from_numpy(A), hk.DeviceBuffer.from_numpy(Bh), hk.DeviceBuffer(M * N * 4)
        none = hk.ptr_array([])
        if packed_first and layout == 0:
            # a packed copy of OTHER values first: the run below hands its own B over and must use that one, and a
            # run without B afterwards must still find the packed values
            other = hk.DeviceBuffer.from_numpy(np.ones_like(Bh))
            hk.check(hk.lib().pml_hip_gemm_pack_b(plan, other.ptr, None))
        hk.check(hk.lib().pml_hip_gemm_invoke(plan, dA.ptr, dB.ptr, dC.ptr, None, none, none, None))
        hk.check(hk.lib().pml_hip_stream_sync(None))
        out.append(dC.to_numpy(np.float32, (M, N)))
        if packed_first and layout == 0:
            hk.check(hk.lib().pml_hip_gemm_invoke(plan, dA.ptr, None, dC.ptr, None, none, none, None))
            hk.check(hk.lib().pml_hip_stream_sync(None))
            ones = dC.to_numpy(np.float32, (M, N))
            np.testing.assert_allclose(ones, np.repeat(A.astype(np.float64).sum(axis=1)[:, None], N, axis=1), rtol=1e-3, atol=1e-3)
        hk.lib().pml_hip_plan_free(plan)
    return out


@pytest.mark.gpu
@pytest.mark.parametrize('flags', [0, hk.FP32_AS_BF16X3])
@pytest.mark.parametrize('M,N,K,ldb', [(1024, 1024, 1024, 1024), (100, 68, 72, 72), (64, 64, 36, 64), (200, 260, 132, 300),
                                       (130, 4, 8, 4), (96, 512, 2048, 516), (77, 66, 40, 66)])
def test_gemm_f32_right_hand_side_as_given(M, N, K, ldb, flags):
    """An fp32 [K][N] right-hand side that arrives with the call is read where it lies (no transposed copy): the
    result has the same bits as the one from the same values in [N][K] layout -- the two differ only in how the
    fragments reach the registers, not in what is multiplied or in which order it is summed -- and agrees with
    float64.  Ragged last tiles in N and K, a leading dimension wider than N with NaNs in the gap, a K
    of one short slab, and (N = 66) a shape that falls back to the transposed copy."""
    print('fp32 right-hand side as given', (M, N, K, ldb, flags), flush=True)
    rng = np.random.default_rng(M * 7 + N + K)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (K, N)).astype(np.float32)
    as_given, n_major = _gemm_f32_layouts(A, B, ldb, flags, packed_first=(M == 100))
    np.testing.assert_array_equal(as_given.view(np.uint32), n_major.view(np.uint32))
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(as_given, ref, rtol=FP32_RTOL if not flags else 1e-3, atol=1e-4 if not flags else 2e-3)


@pytest.mark.gpu
@pytest.mark.parametrize('M,N,K,ldb', [(512, 4096, 4096, 4096), (100, 64, 48, 80), (257, 144, 1040, 160), (64, 16, 16, 16),
                                       (4096, 1024, 2048, 1024)])
def test_gemm_int8_right_hand_side_as_given(M, N, K, ldb):
    """An int8 [K][N] right-hand side whose rows are whole 16-byte vectors is read where it lies (K-values gathered by
    transposing LDS reads) as long as a transposed copy would cost more than the slower reads: bit for bit the int64
    product, with a leading dimension wider than N whose gap holds values that must not be read, ragged tiles in
    M, N and K, and (the last case) a problem large enough to take the transposed copy instead."""
    print('int8 right-hand side as given', (M, N, K, ldb), flush=True)
    rng = np.random.default_rng(M + N + K)
    A = rng.integers(-127, 128, (M, K), dtype=np.int8)
    Bh = rng.integers(-127, 128, (K, ldb), dtype=np.int8)
    d = hk.GemmDesc()
    d.in_dtype, d.out_dtype, d.c_dtype = hk.I8, hk.I32, hk.I32
    d.m, d.n, d.k, d.lda, d.ldb, d.ldc = M, N, K, K, ldb, N
    plan = hk.lib().pml_hip_gemm_dispatch(ctypes.byref(d))
    assert plan, hk.lib().pml_hip_last_error()
    dA, dB, dC = hk.DeviceBuffer.from_numpy(A), hk.DeviceBuffer.from_numpy(Bh), hk.DeviceBuffer(M * N * 4)
    none = hk.ptr_array([])
    hk.check(hk.lib().pml_hip_gemm_invoke(plan, dA.ptr, dB.ptr, dC.ptr, None, none, none, None))
    hk.check(hk.lib().pml_hip_stream_sync(None))
    got = dC.to_numpy(np.int32, (M, N))
    hk.lib().pml_hip_plan_free(plan)
    # (float64 holds these sums exactly -- |sum| <= 127^2 K < 2^53 -- and multiplies through BLAS)
    want = (A.astype(np.float64) @ Bh[:, :N].astype(np.float64)).astype(np.int64).astype(np.int32)
    np.testing.assert_array_equal(got, want)


MANY_ROWS_CASES = [(140837, 128, 64), (70000, 256, 136), (140800, 128, 256)]


@pytest.mark.gpu
@pytest.mark.parametrize('M,N,K', MANY_ROWS_CASES)
def test_gemm_many_rows_short_k(M, N, K):
    """The shape class of a residual network's 1x1 convolutions -- a hundred thousand rows and more, K of one to
    four slabs, thousands of tiles: small-integer operands make every sum exact, so all four vector tails are pinned
    bit for bit by the step semantics, on a ragged last row tile as well."""
    print('many rows, short K', (M, N, K), flush=True)
    rng = np.random.default_rng(M + K)
    A = rng.integers(-4, 5, (M, K)).astype(np.float32)
    B = rng.integers(-4, 5, (K, N)).astype(np.float32)
    bias = E.round_bf16(rng.standard_normal(N).astype(np.float32) * 8)
    scale = E.round_bf16(rng.uniform(0.5, 1.5, N).astype(np.float32))
    shift = E.round_bf16(rng.standard_normal(N).astype(np.float32) * 20)
    res = E.round_bf16(rng.standard_normal((M, N)).astype(np.float32) * 30)
    prod = A @ B
    np.testing.assert_array_equal(run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16), bf16(E.round_bf16(prod)))
    x = E.round_bf16(prod + bias)
    tail = hk.make_tail(ops=[(hk.EPI_RELU, hk.BF16, 0, 0, 0.0)], operands=[])
    C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail)
    np.testing.assert_array_equal(C, bf16(np.maximum(x, 0)))
    tail = hk.make_tail(ops=[(hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_RELU, hk.BF16, 0, 0, 0.0)], operands=[(hk.BF16, N, 1)])
    C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail, operands=(bf16(res),))
    np.testing.assert_array_equal(C, bf16(np.maximum(E.round_bf16(x + res), 0)))
    tail = hk.make_tail(ops=[(hk.EPI_MUL, hk.BF16, hk.OPND_TENSOR, 0, 0.0), (hk.EPI_ADD, hk.BF16, hk.OPND_TENSOR, 1, 0.0)],
                        operands=[(hk.BF16, 0, 1), (hk.BF16, 0, 1)])
    C = run_gemm(bf16(A), bf16(B), hk.BF16, hk.BF16, init=bf16(bias), init_strides=(0, 1), init_dt=hk.BF16, tail=tail,
                 operands=(bf16(scale), bf16(shift)))
    np.testing.assert_array_equal(C, bf16(E.round_bf16(E.round_bf16(x * scale) + shift)))

"""pml_hip_gemm_run_static -- the GEMM entry point that allocates nothing (its transposed right-hand side lives
in a fixed array of the library's device image) -- against pml_hip_gemm_dispatch + pml_hip_gemm_invoke, through
the C ABI: int8 -> int32 bit for bit, bf16 bit for bit (same tile choice, same kernels), two calls in a row, the
second on a smaller problem, and the size limit.  Which cases pass through the array: bf16 always; fp32 only when the
right-hand side cannot be read where it lies (rows that are not whole 16-byte vectors: the `f32_ragged` case); int8
when the transposed copy is cheaper than transposing reads (a tall problem, `i8_tall`) or its rows are ragged (the
second `i8` size).  For those the array keeps the first call's contents when the second, smaller call begins.  The
"allocates nothing" claim is checked against the device's free memory before and after the call."""
import ctypes

import numpy as np
import pytest

from plaidml_amd import hipkernels as hk

STATIC_SCRATCH_BYTES = 32 * 1024 * 1024  # PML_HIP_STATIC_SCRATCH_BYTES


def _desc(kind, m, n, k):
    d = hk.GemmDesc()
    if kind.startswith('i8'):
        d.in_dtype, d.out_dtype, d.c_dtype = hk.I8, hk.I32, hk.I32
    elif kind == 'bf16':
        d.in_dtype, d.out_dtype, d.c_dtype = hk.BF16, hk.BF16, hk.BF16
    else:
        d.in_dtype, d.out_dtype, d.c_dtype = hk.F32, hk.F32, hk.F32
    d.m, d.n, d.k, d.lda, d.ldb, d.ldc = m, n, k, k, n, n
    d.b_layout = 0  # B is [K][N]: both entry points transpose it before the matrix-core kernel
    return d


def _inputs(kind, m, n, k, seed):
    r = np.random.default_rng(seed)
    if kind.startswith('i8'):
        return r.integers(-127, 128, (m, k), dtype=np.int8), r.integers(-127, 128, (k, n), dtype=np.int8), np.int32
    if kind == 'bf16':
        bits = lambda a: (a.astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)  # noqa: E731  (truncation: any bf16 value will do)
        return bits(r.standard_normal((m, k))), bits(r.standard_normal((k, n))), np.uint16
    return r.standard_normal((m, k)).astype(np.float32), r.standard_normal((k, n)).astype(np.float32), np.float32


def _free_device_bytes():
    """hipMemGetInfo of the current device, straight from the HIP runtime the kernel library has loaded."""
    hip = ctypes.CDLL('libamdhip64.so')
    free, total = ctypes.c_size_t(), ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free), ctypes.byref(total)) == 0
    return free.value


def _both(kind, m, n, k, seed):
    L = hk.lib()
    none = hk.ptr_array([])
    a, b, out_t = _inputs(kind, m, n, k, seed)
    d = _desc(kind, m, n, k)
    dA, dB = hk.DeviceBuffer.from_numpy(a), hk.DeviceBuffer.from_numpy(b)
    nbytes = m * n * np.dtype(out_t).itemsize
    dC1, dC2 = hk.DeviceBuffer(nbytes), hk.DeviceBuffer(nbytes)
    hk.check(L.pml_hip_fill_u32(dC1.ptr, 0xdeadbeef, nbytes // 4, None))
    hk.check(L.pml_hip_fill_u32(dC2.ptr, 0x0badf00d, nbytes // 4, None))
    plan = L.pml_hip_gemm_dispatch(ctypes.byref(d))
    assert plan, L.pml_hip_last_error()
    hk.check(L.pml_hip_gemm_invoke(plan, dA.ptr, dB.ptr, dC1.ptr, None, none, none, None))
    hk.check(L.pml_hip_stream_sync(None))
    free_before = _free_device_bytes()
    hk.check(L.pml_hip_gemm_run_static(ctypes.byref(d), dA.ptr, dB.ptr, dC2.ptr, None, none, none, None))
    hk.check(L.pml_hip_stream_sync(None))
    assert _free_device_bytes() == free_before, 'pml_hip_gemm_run_static changed the amount of free device memory'
    c1, c2 = dC1.to_numpy(out_t, (m, n)), dC2.to_numpy(out_t, (m, n))
    L.pml_hip_plan_free(plan)
    return a, b, c1, c2


# first call: a right-hand side that fills a good part of the array; second: a smaller one, ragged in m and n
SIZES = {'i8': ((512, 1024, 2048), (200, 136, 320)), 'bf16': ((512, 1024, 2048), (200, 136, 320)),
         'f32': ((512, 1024, 2048), (200, 136, 320)),
         # n % 4 != 0: the fp32 right-hand side cannot be read where it lies and is transposed into the array
         'f32_ragged': ((512, 1022, 2048), (200, 134, 320)),
         # 8192 rows: the transposed copy (into the array) costs less than transposing LDS reads would
         'i8_tall': ((8192, 2048, 2048), (8000, 1936, 2048))}


@pytest.mark.gpu
@pytest.mark.parametrize('kind', ['i8', 'bf16', 'f32', 'f32_ragged', 'i8_tall'])
def test_static_scratch_gemm_equals_the_plan_based_one_twice_in_a_row(kind):
    hk.init(0)
    print('gemm_run_static', kind, flush=True)
    for (m, n, k), seed in zip(SIZES[kind], (1, 2)):
        a, b, c1, c2 = _both(kind, m, n, k, seed)
        np.testing.assert_array_equal(c2, c1)
        if kind.startswith('i8'):  # and both are right
            np.testing.assert_array_equal(c1[:8], a[:8].astype(np.int32) @ b.astype(np.int32))


def test_static_scratch_gemm_rejects_what_does_not_fit():
    """No GPU needed: the descriptor is rejected before anything touches the device."""
    L = hk.lib()
    one = ctypes.c_void_p(256)   # never dereferenced
    d = _desc('bf16', 128, 4096, 4096 + 8)  # 4096 x 4104 x 2 bytes > 32 MiB
    assert 4096 * 4104 * 2 > STATIC_SCRATCH_BYTES
    assert L.pml_hip_gemm_run_static(ctypes.byref(d), one, one, one, None, hk.ptr_array([]), hk.ptr_array([]), None) != 0
    assert b'PML_HIP_STATIC_SCRATCH_BYTES' in L.pml_hip_last_error()
    d = _desc('i8', 128, 64, 64)
    assert L.pml_hip_gemm_run_static(ctypes.byref(d), one, None, one, None, hk.ptr_array([]), hk.ptr_array([]), None) != 0
    assert b'b is null' in L.pml_hip_last_error()

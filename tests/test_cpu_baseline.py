"""The OpenMP CPU baseline computes the same contraction as the generic oracle."""
import ctypes
import os

import numpy as np

from oracle import tile_oracle as E
from oracle import tile_oplib as op

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def lib():
    return ctypes.CDLL(os.path.join(ROOT, 'oracle', 'libcpu_baseline.so'))


def test_conv_baseline_matches_oracle():
    rng = np.random.default_rng(0)
    Iv = rng.standard_normal((2, 9, 9, 8)).astype(np.float32)
    Fv = rng.standard_normal((3, 3, 8, 16)).astype(np.float32)
    bias = rng.standard_normal(16).astype(np.float32)
    out = np.empty((2, 9, 9, 16), np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    lib().cpu_conv2d_nhwc_f32(Iv.ctypes.data_as(fp), Fv.ctypes.data_as(fp), bias.ctypes.data_as(fp),
                              out.ctypes.data_as(fp), 2, 9, 9, 8, 3, 3, 16, 9, 9, 1, 1, 1)
    I, F, B = E.Placeholder(E.DType.FLOAT32, Iv.shape), E.Placeholder(E.DType.FLOAT32, Fv.shape), E.Placeholder(E.DType.FLOAT32, [16])
    ref, = E.run(E.Program('c', [I, F, B], [op.relu(op.convolution(I, F) + B)]), [Iv, Fv, bias])
    np.testing.assert_allclose(out, ref, rtol=1e-5, atol=1e-5)


def test_gemm_baselines_match_numpy():
    rng = np.random.default_rng(1)
    A = rng.standard_normal((17, 33)).astype(np.float32)
    B = rng.standard_normal((33, 9)).astype(np.float32)
    C = np.empty((17, 9), np.float32)
    fp = ctypes.POINTER(ctypes.c_float)
    lib().cpu_gemm_f32(A.ctypes.data_as(fp), B.ctypes.data_as(fp), C.ctypes.data_as(fp), 17, 9, 33)
    np.testing.assert_allclose(C, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-5, atol=1e-5)
    Ai = rng.integers(-127, 128, (17, 33), dtype=np.int8)
    Bi = rng.integers(-127, 128, (33, 9), dtype=np.int8)
    Ci = np.empty((17, 9), np.int32)
    lib().cpu_gemm_i8_i32(Ai.ctypes.data_as(ctypes.c_void_p), Bi.ctypes.data_as(ctypes.c_void_p),
                          Ci.ctypes.data_as(ctypes.c_void_p), 17, 9, 33)
    np.testing.assert_array_equal(Ci, Ai.astype(np.int32) @ Bi.astype(np.int32))

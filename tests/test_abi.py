"""The C-ABI libraries load and export every symbol their headers declare (no GPU needed)."""
import ctypes
import os
import re

from plaidml_amd import hipkernels as hk

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header):
    text = open(os.path.join(ROOT, 'include', header)).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(pml_hip_[a-z0-9_]+)\s*\(', text)))


def test_kernel_library_exports_every_declared_symbol():
    names = declared('pml_hip.h')
    assert len(names) >= 30
    L = hk.lib()
    for n in names:
        assert hasattr(L, n), n
    assert sorted(hk.EXPORTS) == names


def test_descriptor_layouts_match():
    L = hk.lib()
    for which, cls in enumerate([hk.Epilogue, hk.GemmDesc, hk.Conv2dDesc, hk.Dwconv2dDesc, hk.Pool2dDesc,
                                 hk.EltwiseDesc, hk.SelectDesc, hk.ContractDesc, hk.Form, hk.GatherDesc, hk.ScatterDesc,
                                 hk.ArgsortDesc, hk.SoftmaxDesc]):
        assert L.pml_hip_struct_size(which) == ctypes.sizeof(cls), cls.__name__


def test_dispatch_rejects_bad_descriptors_without_a_gpu():
    L = hk.lib()
    d = hk.GemmDesc()
    d.in_dtype, d.out_dtype = hk.F64, hk.F64
    assert L.pml_hip_gemm_dispatch(ctypes.byref(d)) == 0
    assert b'in_dtype' in L.pml_hip_last_error()
    c = hk.Conv2dDesc()
    c.in_dtype, c.out_dtype = hk.BF16, hk.BF16
    assert L.pml_hip_conv2d_dispatch(ctypes.byref(c)) == 0
    assert b'geometry' in L.pml_hip_last_error()
    g = hk.GatherDesc()
    g.rank, g.idx_rank, g.dtype, g.idx_dtype, g.axis = 1, 1, hk.F32, hk.I32, 3
    one = ctypes.c_void_p(1)   # never dereferenced: the descriptor is rejected first
    assert L.pml_hip_gather(ctypes.byref(g), one, one, one, None) != 0
    assert b'axis out of range' in L.pml_hip_last_error()
    sc = hk.ScatterDesc()
    sc.rank, sc.idx_rank, sc.upd_rank, sc.dtype, sc.idx_dtype = 1, 1, 1, hk.F32, hk.F32
    assert L.pml_hip_scatter(ctypes.byref(sc), one, ctypes.c_void_p(2), one, ctypes.c_void_p(3), None) != 0
    assert b'si32 or ui32' in L.pml_hip_last_error()
    # an elementwise chain whose step names an operand outside the operand list
    e = hk.EltwiseDesc()
    e.rank = 1
    e.tail = hk.make_tail(ops=[(hk.EPI_ADD, hk.F32, hk.OPND_TENSOR, 3, 0.0)], operands=[(hk.F32, 0, 1)])
    assert L.pml_hip_eltwise_dispatch(ctypes.byref(e)) == 0
    assert b'outside the operand list' in L.pml_hip_last_error()
    # a pooling divisor goes with the sum over a whole image only
    p = hk.Pool2dDesc()
    p.dtype, p.agg = hk.BF16, hk.AGG_ADD
    p.n, p.h, p.w, p.c, p.kh, p.kw, p.oh, p.ow = 1, 8, 8, 16, 2, 2, 4, 4
    p.stride_h = p.stride_w = 2
    p.divisor = 4.0
    assert L.pml_hip_pool2d_dispatch(ctypes.byref(p)) == 0
    assert b'divisor' in L.pml_hip_last_error()
    p.kh = p.kw = 8
    p.oh = p.ow = p.stride_h = p.stride_w = 1
    p.agg = hk.AGG_MAX
    assert L.pml_hip_pool2d_dispatch(ctypes.byref(p)) == 0
    p.agg = hk.AGG_ADD
    plan = L.pml_hip_pool2d_dispatch(ctypes.byref(p))
    assert plan, L.pml_hip_last_error()
    L.pml_hip_plan_free(plan)

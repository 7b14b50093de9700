"""ctypes view of the kernel library's C ABI (include/pml_hip.h).

Loads plaidml_amd/lib/libpml_hip.so, which must have been built beforehand
(`python -c "import __graft_entry__ as g; g.build()"` or `make -C plaidml_amd/csrc`).
There is no fallback: a missing library or a missing GPU raises.
"""
import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libpml_hip.so')

# element types (values of plaidml_datatype, bfloat16 appended)
BOOL, I8, U8, I16, U16, I32, U32, I64, U64, F16, F32, F64, BF16 = 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16
FP32_AS_BF16X3 = 1  # descriptor flag of gemm / conv2d: fp32 operands multiplied as three bf16 products
# schedule overrides in the same `flags` field (PML_HIP_FLAG_TILE / PML_HIP_FLAG_CONV of include/pml_hip.h)
TILE_NAMES = ('64x64', '128x64', '128x128', '128x64w8', '128x128w8', '256x128w16', '128x128w8s2', '64x64w8k2', '256x256w8', '128x64n2', '192x384w8', '64x64ks')
CONV_AUTO, CONV_IGEMM, CONV_PATCHES, CONV_LDSFILTER, CONV_BLOCKS = 0, 1, 2, 3, 4


def flag_tile(name):
    """The descriptor bits that name output tile `name` (one of TILE_NAMES)."""
    return (TILE_NAMES.index(name) + 1) << 8


def flag_conv(path):
    """The descriptor bits that name a convolution path (CONV_*)."""
    return path << 16


def flag_maxpool3x3s2(pad_top, pad_bottom, pad_left, pad_right):
    """The conv2d descriptor bits that ask for a 3x3 stride-2 max-pool over the convolution's result inside the launch
    (padding 0 or 1 per side; PML_HIP_FLAG_MAXPOOL3x3S2)."""
    return (1 << 20) | (pad_top & 1) << 21 | (pad_bottom & 1) << 22 | (pad_left & 1) << 23 | (pad_right & 1) << 24

AGG_ASSIGN, AGG_ADD, AGG_MAX, AGG_MIN, AGG_MUL = 0, 1, 2, 3, 4
COMBO_NONE, COMBO_ADD, COMBO_COND, COMBO_EQ, COMBO_MUL = 0, 1, 2, 3, 4
(EPI_ADD, EPI_SUB, EPI_RSUB, EPI_MUL, EPI_DIV, EPI_RDIV, EPI_MAX, EPI_MIN, EPI_RELU, EPI_NEG, EPI_EXP, EPI_LOG,
 EPI_SQRT, EPI_TANH, EPI_FLOOR, EPI_CEIL, EPI_ROUND, EPI_CAST, EPI_STORE, EPI_CMP_LT, EPI_CMP_GT, EPI_CMP_LE,
 EPI_CMP_GE, EPI_CMP_EQ, EPI_CMP_NE, EPI_MAX_GT) = range(1, 27)
OPND_NONE, OPND_IMM, OPND_TENSOR = 0, 1, 2
MAX_EPI_OPS, MAX_EPI_OPERANDS, MAX_RANK, MAX_IDX, MAX_FORMS = 12, 6, 6, 12, 32

EXPORTS = [
    'pml_hip_init', 'pml_hip_device_count', 'pml_hip_device_name', 'pml_hip_last_error', 'pml_hip_malloc',
    'pml_hip_free', 'pml_hip_host_alloc', 'pml_hip_host_free', 'pml_hip_memcpy_h2d', 'pml_hip_memcpy_d2h',
    'pml_hip_memcpy_d2d', 'pml_hip_fill_u32', 'pml_hip_stream_create', 'pml_hip_stream_destroy',
    'pml_hip_stream_sync', 'pml_hip_event_create', 'pml_hip_event_destroy', 'pml_hip_event_record',
    'pml_hip_event_sync', 'pml_hip_event_elapsed_ms', 'pml_hip_capture_begin', 'pml_hip_capture_end',
    'pml_hip_graph_launch', 'pml_hip_graph_destroy', 'pml_hip_gemm_dispatch', 'pml_hip_gemm_invoke',
    'pml_hip_gemm_run_static', 'pml_hip_gemm_invoke2', 'pml_hip_gemm_pack_b2', 'pml_hip_probe_mfma', 'pml_hip_dwconv2d_pack_filter', 'pml_hip_tile_of_workgroup', 'pml_hip_tile_name', 'pml_hip_tile_by_name', 'pml_hip_gemm_tail_cheaper_apart',
    'pml_hip_conv2d_dispatch', 'pml_hip_conv2d_invoke', 'pml_hip_dwconv2d_dispatch', 'pml_hip_dwconv2d_invoke',
    'pml_hip_pool2d_dispatch', 'pml_hip_pool2d_invoke', 'pml_hip_eltwise_dispatch', 'pml_hip_eltwise_invoke',
    'pml_hip_select', 'pml_hip_softmax', 'pml_hip_index', 'pml_hip_contract_dispatch', 'pml_hip_contract_invoke', 'pml_hip_plan_free',
    'pml_hip_plan_describe', 'pml_hip_struct_size', 'pml_hip_gemm_pack_b', 'pml_hip_conv2d_pack_filter', 'pml_hip_conv2d_takes_maxpool',
    'pml_hip_gather', 'pml_hip_scatter', 'pml_hip_argsort', 'pml_hip_prng',
]

i32, i64, f64 = ctypes.c_int32, ctypes.c_int64, ctypes.c_double


class EpiOp(ctypes.Structure):
    _fields_ = [('opcode', i32), ('dtype', i32), ('operand_kind', i32), ('operand', i32), ('imm', f64)]


class Epilogue(ctypes.Structure):
    _fields_ = [('n_ops', i32), ('n_operands', i32), ('ops', EpiOp * MAX_EPI_OPS),
                ('operand_dtype', i32 * MAX_EPI_OPERANDS), ('operand_row_stride', i64 * MAX_EPI_OPERANDS),
                ('operand_col_stride', i64 * MAX_EPI_OPERANDS)]


class GemmDesc(ctypes.Structure):
    _fields_ = [('in_dtype', i32), ('out_dtype', i32), ('m', i64), ('n', i64), ('k', i64), ('lda', i64), ('ldb', i64),
                ('ldc', i64), ('init_kind', i32), ('init_dtype', i32), ('init_row_stride', i64),
                ('init_col_stride', i64), ('c_dtype', i32), ('b_layout', i32), ('tail', Epilogue),
                ('k2', i64), ('lda2', i64), ('ldb2', i64), ('a2_stride', i32), ('init2_kind', i32),
                ('a2_h', i64), ('a2_w', i64), ('a2_oh', i64), ('a2_ow', i64), ('flags', i32), ('reserved', i32)]


class Conv2dDesc(ctypes.Structure):
    _fields_ = [('in_dtype', i32), ('out_dtype', i32), ('n', i64), ('h', i64), ('w', i64), ('ci', i64), ('kh', i64),
                ('kw', i64), ('co', i64), ('oh', i64), ('ow', i64), ('stride_h', i64), ('stride_w', i64),
                ('dil_h', i64), ('dil_w', i64), ('pad_h', i64), ('pad_w', i64), ('init_kind', i32),
                ('init_dtype', i32), ('init_row_stride', i64), ('init_col_stride', i64), ('c_dtype', i32),
                ('flags', i32), ('tail', Epilogue)]


class Dwconv2dDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('out_pitch', i32), ('n', i64), ('h', i64), ('w', i64), ('c', i64), ('kh', i64),
                ('kw', i64), ('oh', i64), ('ow', i64), ('stride_h', i64), ('stride_w', i64), ('dil_h', i64),
                ('dil_w', i64), ('pad_h', i64), ('pad_w', i64), ('tail', Epilogue)]


class Pool2dDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('agg', i32), ('n', i64), ('h', i64), ('w', i64), ('c', i64), ('kh', i64), ('kw', i64),
                ('oh', i64), ('ow', i64), ('stride_h', i64), ('stride_w', i64), ('pad_h', i64), ('pad_w', i64),
                ('with_index', i32), ('divisor', ctypes.c_float)]


class EltwiseDesc(ctypes.Structure):
    _fields_ = [('rank', i32), ('in_dtype', i32), ('out_dtype', i32), ('reserved', i32), ('sizes', i64 * MAX_RANK),
                ('in_strides', i64 * MAX_RANK), ('operand_strides', (i64 * MAX_RANK) * MAX_EPI_OPERANDS),
                ('tail', Epilogue)]


class SelectDesc(ctypes.Structure):
    _fields_ = [('rank', i32), ('cond_dtype', i32), ('t_dtype', i32), ('f_dtype', i32), ('out_dtype', i32),
                ('reserved', i32), ('sizes', i64 * MAX_RANK), ('cond_strides', i64 * MAX_RANK),
                ('t_strides', i64 * MAX_RANK), ('f_strides', i64 * MAX_RANK)]


class Form(ctypes.Structure):
    _fields_ = [('coef', i32 * MAX_IDX), ('c0', i32), ('den', i32), ('operand', i32), ('size', i64), ('stride', i64)]


class ContractDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('agg', i32), ('combo', i32), ('n_idx', i32), ('n_out_idx', i32), ('n_src', i32),
                ('n_forms', i32), ('cmp_dtype', i32), ('src_dtype', i32 * 3), ('has_init', i32),
                ('lo', i64 * MAX_IDX), ('hi', i64 * MAX_IDX), ('out_elems', i64), ('identity_f', f64),
                ('identity_i', i64), ('forms', Form * MAX_FORMS)]


MAX_SPECIAL_RANK = 8


class GatherDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('idx_dtype', i32), ('mode', i32), ('interpolation', i32), ('nearest', i32), ('oob', i32),
                ('axis', i32), ('batch_dims', i32), ('rank', i32), ('idx_rank', i32), ('cube_coeff', f64),
                ('sizes', i64 * MAX_SPECIAL_RANK), ('idx_sizes', i64 * MAX_SPECIAL_RANK)]


class ScatterDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('idx_dtype', i32), ('mode', i32), ('axis', i32), ('rank', i32), ('idx_rank', i32),
                ('upd_rank', i32), ('reserved', i32), ('sizes', i64 * MAX_SPECIAL_RANK), ('idx_sizes', i64 * MAX_SPECIAL_RANK),
                ('upd_sizes', i64 * MAX_SPECIAL_RANK)]


class ArgsortDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('rank', i32), ('axis', i32), ('direction', i32), ('sizes', i64 * MAX_SPECIAL_RANK)]


class SoftmaxDesc(ctypes.Structure):
    _fields_ = [('dtype', i32), ('reserved', i32), ('rows', i64), ('cols', i64)]


_lib = None


def lib():
    """The loaded library.  Raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError('%s is missing: build the HIP kernel library first (there is no CPU fallback)' % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        L.pml_hip_last_error.restype = ctypes.c_char_p
        for name in ('pml_hip_gemm_dispatch', 'pml_hip_conv2d_dispatch', 'pml_hip_dwconv2d_dispatch',
                     'pml_hip_pool2d_dispatch', 'pml_hip_eltwise_dispatch', 'pml_hip_contract_dispatch'):
            getattr(L, name).restype = ctypes.c_int64
        vp, sz = ctypes.c_void_p, ctypes.c_size_t
        L.pml_hip_malloc.argtypes = [ctypes.POINTER(vp), sz]
        L.pml_hip_free.argtypes = [vp]
        L.pml_hip_memcpy_h2d.argtypes = [vp, vp, sz, vp]
        L.pml_hip_memcpy_d2h.argtypes = [vp, vp, sz, vp]
        L.pml_hip_memcpy_d2d.argtypes = [vp, vp, sz, vp]
        L.pml_hip_fill_u32.argtypes = [vp, ctypes.c_uint32, sz, vp]
        L.pml_hip_stream_sync.argtypes = [vp]
        L.pml_hip_event_create.argtypes = [ctypes.POINTER(vp)]
        L.pml_hip_event_destroy.argtypes = [vp]
        L.pml_hip_event_record.argtypes = [vp, vp]
        L.pml_hip_event_sync.argtypes = [vp]
        L.pml_hip_event_elapsed_ms.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_float)]
        L.pml_hip_capture_begin.argtypes = [vp]
        L.pml_hip_capture_end.argtypes = [vp, ctypes.POINTER(vp)]
        L.pml_hip_graph_launch.argtypes = [vp, vp]
        L.pml_hip_graph_destroy.argtypes = [vp]
        pp = ctypes.POINTER(vp)
        L.pml_hip_gemm_invoke.argtypes = [ctypes.c_int64, vp, vp, vp, vp, pp, pp, vp]
        L.pml_hip_gemm_run_static.argtypes = [ctypes.POINTER(GemmDesc), vp, vp, vp, vp, pp, pp, vp]
        L.pml_hip_gemm_invoke2.argtypes = [ctypes.c_int64, vp, vp, vp, vp, vp, vp, vp, pp, pp, vp]
        L.pml_hip_gemm_pack_b2.argtypes = [ctypes.c_int64, vp, vp]
        L.pml_hip_probe_mfma.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
        L.pml_hip_tile_name.restype = ctypes.c_char_p
        L.pml_hip_tile_name.argtypes = [ctypes.c_int]
        L.pml_hip_tile_by_name.argtypes = [ctypes.c_char_p]
        L.pml_hip_tile_of_workgroup.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.pml_hip_gemm_tail_cheaper_apart.argtypes = [ctypes.POINTER(GemmDesc)]
        L.pml_hip_conv2d_invoke.argtypes = [ctypes.c_int64, vp, vp, vp, vp, pp, pp, vp]
        L.pml_hip_dwconv2d_invoke.argtypes = [ctypes.c_int64, vp, vp, vp, pp, pp, vp]
        L.pml_hip_pool2d_invoke.argtypes = [ctypes.c_int64, vp, vp, vp, vp]
        L.pml_hip_eltwise_invoke.argtypes = [ctypes.c_int64, vp, vp, pp, pp, vp]
        L.pml_hip_select.argtypes = [ctypes.POINTER(SelectDesc), vp, vp, vp, vp, vp]
        L.pml_hip_softmax.argtypes = [ctypes.POINTER(SoftmaxDesc), vp, vp, vp]
        L.pml_hip_index.argtypes = [vp, i32, ctypes.POINTER(i64), i32, vp]
        L.pml_hip_contract_invoke.argtypes = [ctypes.c_int64, pp, vp, vp]
        L.pml_hip_plan_free.argtypes = [ctypes.c_int64]
        L.pml_hip_plan_describe.argtypes = [ctypes.c_int64, ctypes.c_char_p, sz]
        L.pml_hip_struct_size.restype = sz
        L.pml_hip_gemm_pack_b.argtypes = [ctypes.c_int64, vp, vp]
        L.pml_hip_gather.argtypes = [ctypes.POINTER(GatherDesc), vp, vp, vp, vp]
        L.pml_hip_scatter.argtypes = [ctypes.POINTER(ScatterDesc), vp, vp, vp, vp, vp]
        L.pml_hip_argsort.argtypes = [ctypes.POINTER(ArgsortDesc), vp, vp, vp]
        L.pml_hip_prng.argtypes = [vp, ctypes.c_int64, vp, vp, vp]
        L.pml_hip_conv2d_pack_filter.argtypes = [ctypes.c_int64, vp, vp]
        L.pml_hip_conv2d_takes_maxpool.argtypes = [vp]
        L.pml_hip_conv2d_takes_maxpool.restype = ctypes.c_int
        L.pml_hip_dwconv2d_pack_filter.argtypes = [ctypes.c_int64, vp, vp]
        _lib = L
    return _lib


class HipError(RuntimeError):
    pass


def check(status):
    if status != 0:
        raise HipError(lib().pml_hip_last_error().decode())


def init(device=0):
    check(lib().pml_hip_init(device))


def device_name():
    buf = ctypes.create_string_buffer(256)
    check(lib().pml_hip_device_name(buf, 256))
    return buf.value.decode()


class DeviceBuffer:
    """A device allocation with numpy upload / download helpers."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = ctypes.c_void_p()
        check(lib().pml_hip_malloc(ctypes.byref(p), self.nbytes))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        if a.nbytes:
            check(lib().pml_hip_memcpy_h2d(b.ptr, a.ctypes.data, a.nbytes, None))
        return b

    def to_numpy(self, dtype, shape):
        out = np.empty(shape, dtype=dtype)
        if out.nbytes:
            check(lib().pml_hip_memcpy_d2h(out.ctypes.data, self.ptr, out.nbytes, None))
        return out

    def fill_u32(self, pattern):
        check(lib().pml_hip_fill_u32(self.ptr, pattern, self.nbytes // 4, None))

    def free(self):
        if self.ptr:
            lib().pml_hip_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def make_tail(ops=(), operands=()):
    """ops: (opcode, dtype, kind, operand, imm); operands: (dtype, row_stride, col_stride)."""
    t = Epilogue()
    t.n_ops = len(ops)
    t.n_operands = len(operands)
    for i, (opc, dt, kind, opnd, imm) in enumerate(ops):
        t.ops[i] = EpiOp(opc, dt, kind, opnd, imm)
    for i, (dt, rs, cs) in enumerate(operands):
        t.operand_dtype[i] = dt
        t.operand_row_stride[i] = rs
        t.operand_col_stride[i] = cs
    return t


def ptr_array(ptrs, n=MAX_EPI_OPERANDS):
    arr = (ctypes.c_void_p * n)()
    for i, p in enumerate(ptrs):
        arr[i] = p
    return arr


def describe(plan):
    buf = ctypes.create_string_buffer(512)
    check(lib().pml_hip_plan_describe(plan, buf, 512))
    return buf.value.decode()


class Timer:
    """HIP-event timing on a stream (NULL = the stream every invoke here uses)."""

    def __init__(self):
        self.e0, self.e1 = ctypes.c_void_p(), ctypes.c_void_p()
        check(lib().pml_hip_event_create(ctypes.byref(self.e0)))
        check(lib().pml_hip_event_create(ctypes.byref(self.e1)))

    def start(self, stream=None):
        check(lib().pml_hip_event_record(self.e0, stream))

    def stop(self, stream=None):
        check(lib().pml_hip_event_record(self.e1, stream))
        check(lib().pml_hip_event_sync(self.e1))
        ms = ctypes.c_float()
        check(lib().pml_hip_event_elapsed_ms(self.e0, self.e1, ctypes.byref(ms)))
        return ms.value

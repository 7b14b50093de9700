"""Python view of libplaidml.so (the plaidml_* C ABI) through ctypes.

Mirrors the reference's Python packages plaidml.core / plaidml.edsl / plaidml.exec
(plaidml/core/__init__.py:72-330, plaidml/edsl/__init__.py:32-1180,
plaidml/exec/__init__.py:25-70): DType, TensorShape, Buffer, Program, TensorDim,
TensorIndex, Tensor, Contraction, the intrinsics, Executable and run().  The
reference binds the same C functions with cffi; ctypes is used here because cffi is
not available.  Everything executes on the `hip` device: there is no CPU path.
"""
import builtins
import ctypes
import enum
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, 'lib', 'libplaidml.so')

vp, sz, i64, f64 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int64, ctypes.c_double


class Error(ctypes.Structure):
    _fields_ = [('code', sz), ('msg', vp)]


class _List(ctypes.Structure):
    _fields_ = [('size', sz), ('elts', ctypes.POINTER(vp))]


class _Integers(ctypes.Structure):
    _fields_ = [('size', sz), ('elts', ctypes.POINTER(i64))]


class _Kvp(ctypes.Structure):
    _fields_ = [('key', vp), ('value', vp)]


class _Kvps(ctypes.Structure):
    _fields_ = [('size', sz), ('elts', ctypes.POINTER(_Kvp))]


# name -> (restype, argtypes after the leading plaidml_error*)
_SIGS = {
    'plaidml_init': (None, []), 'plaidml_shutdown': (None, []), 'plaidml_version': (ctypes.c_char_p, []),
    'plaidml_integers_free': (None, [vp]), 'plaidml_strings_free': (None, [vp]), 'plaidml_kvps_free': (None, [vp]),
    'plaidml_shapes_free': (None, [vp]),
    'plaidml_settings_list': (ctypes.POINTER(_Kvps), []), 'plaidml_settings_get': (vp, [ctypes.c_char_p]),
    'plaidml_settings_set': (None, [ctypes.c_char_p, ctypes.c_char_p]), 'plaidml_settings_load': (None, []),
    'plaidml_settings_save': (None, []),
    'plaidml_shape_free': (None, [vp]),
    'plaidml_shape_alloc': (vp, [ctypes.c_int, sz, ctypes.POINTER(i64), ctypes.POINTER(i64)]),
    'plaidml_shape_clone': (vp, [vp]), 'plaidml_shape_repr': (vp, [vp]), 'plaidml_shape_get_rank': (sz, [vp]),
    'plaidml_shape_get_dtype': (ctypes.c_int, [vp]), 'plaidml_shape_get_sizes': (ctypes.POINTER(_Integers), [vp]),
    'plaidml_shape_get_strides': (ctypes.POINTER(_Integers), [vp]), 'plaidml_shape_get_nbytes': (ctypes.c_uint64, [vp]),
    'plaidml_buffer_alloc': (vp, [vp]), 'plaidml_buffer_adopt': (vp, [vp, vp, sz]), 'plaidml_buffer_free': (None, [vp]),
    'plaidml_buffer_clone': (vp, [vp]), 'plaidml_buffer_shape': (vp, [vp]), 'plaidml_buffer_data': (vp, [vp]),
    'plaidml_buffer_size': (sz, [vp]),
    'plaidml_program_free': (None, [vp]), 'plaidml_program_repr': (vp, [vp]),
    'plaidml_program_get_inputs': (ctypes.POINTER(_List), [vp]), 'plaidml_program_get_outputs': (ctypes.POINTER(_List), [vp]),
    'plaidml_program_get_passes': (ctypes.POINTER(_Kvps), [vp]),
    'plaidml_program_compile': (None, [vp, ctypes.c_bool, ctypes.c_char_p]),
    'plaidml_program_save': (vp, [vp, sz, vp, vp]),
    'plaidml_edsl_init': (None, []),
    'plaidml_poly_expr_free': (None, [vp]), 'plaidml_poly_expr_repr': (vp, [vp]), 'plaidml_poly_expr_dim': (vp, [vp]),
    'plaidml_poly_expr_index': (vp, [ctypes.c_char_p]), 'plaidml_poly_expr_literal': (vp, [i64]),
    'plaidml_poly_expr_op': (vp, [ctypes.c_int, sz, ctypes.POINTER(vp)]),
    'plaidml_dim_expr_free': (None, [vp]), 'plaidml_dim_expr_repr': (vp, [vp]), 'plaidml_dim_expr_none': (vp, []),
    'plaidml_dim_expr_int': (vp, [i64]), 'plaidml_dim_expr_op': (vp, [ctypes.c_int, sz, ctypes.POINTER(vp)]),
    'plaidml_expr_free': (None, [vp]), 'plaidml_expr_ptr': (vp, [vp]), 'plaidml_expr_get_dtype': (ctypes.c_int, [vp]),
    'plaidml_expr_get_rank': (sz, [vp]), 'plaidml_expr_get_shape': (vp, [vp]),
    'plaidml_expr_bind_dims': (None, [vp, sz, ctypes.POINTER(vp)]), 'plaidml_expr_repr': (vp, [vp]),
    'plaidml_expr_clone': (vp, [vp]), 'plaidml_expr_get_dim': (vp, [vp]), 'plaidml_expr_dim': (vp, [vp]),
    'plaidml_expr_input': (vp, [vp, ctypes.c_char_p]), 'plaidml_expr_constant': (vp, [vp, ctypes.c_char_p]),
    'plaidml_expr_uint': (vp, [ctypes.c_uint64]), 'plaidml_expr_int': (vp, [i64]), 'plaidml_expr_float': (vp, [f64]),
    'plaidml_expr_element': (vp, [vp, sz]),
    'plaidml_expr_intrinsic': (vp, [ctypes.c_char_p, sz, ctypes.POINTER(vp), ctypes.c_char_p]),
    'plaidml_expr_cast': (vp, [vp, ctypes.c_int]), 'plaidml_expr_pragma': (vp, [vp, ctypes.c_char_p, sz, vp]),
    'plaidml_exprs_free': (None, [vp]), 'plaidml_expr_layer_begin': (vp, [ctypes.c_char_p, sz, vp, sz, vp]),
    'plaidml_expr_layer_end': (ctypes.POINTER(_List), [vp, sz, ctypes.POINTER(vp)]),
    'plaidml_expr_contraction': (vp, [ctypes.c_int, ctypes.c_int, sz, ctypes.POINTER(vp), ctypes.POINTER(vp), vp, ctypes.c_char_p]),
    'plaidml_contraction_add_operand': (None, [vp, vp, sz, ctypes.POINTER(vp)]),
    'plaidml_contraction_add_constraint': (None, [vp, vp, vp]), 'plaidml_contraction_build': (None, [vp]),
    'plaidml_tuple_free': (None, [vp]), 'plaidml_value_free': (None, [vp]), 'plaidml_value_clone': (vp, [vp]),
    'plaidml_value_get_kind': (ctypes.c_int, [vp]), 'plaidml_value_none': (vp, []), 'plaidml_value_dim': (vp, [vp]),
    'plaidml_value_expr': (vp, [vp]), 'plaidml_value_float': (vp, [f64]), 'plaidml_value_int': (vp, [i64]),
    'plaidml_value_str': (vp, [ctypes.c_char_p]), 'plaidml_value_tuple': (vp, [sz, ctypes.POINTER(vp)]),
    'plaidml_value_dim_get': (vp, [vp]), 'plaidml_value_expr_get': (vp, [vp]), 'plaidml_value_float_get': (f64, [vp]),
    'plaidml_value_int_get': (i64, [vp]), 'plaidml_value_str_get': (vp, [vp]),
    'plaidml_value_tuple_get': (ctypes.POINTER(_List), [vp]), 'plaidml_value_repr': (vp, [vp]),
    'plaidml_targets_get': (ctypes.POINTER(_List), []),
    'plaidml_build': (vp, [ctypes.c_char_p, sz, ctypes.POINTER(vp), vp, sz, ctypes.POINTER(vp)]),
    'plaidml_op_make': (vp, [ctypes.c_char_p, vp]),
    'plaidml_exec_init': (None, []), 'plaidml_devices_get': (ctypes.POINTER(_List), []),
    'plaidml_jit': (vp, [vp, ctypes.c_char_p]), 'plaidml_executable_free': (None, [vp]),
    'plaidml_executable_run': (f64, [vp, sz, ctypes.POINTER(vp), sz, ctypes.POINTER(vp)]),
}
# the two functions that take no plaidml_error, and the statistics helper
EXPORTS = sorted(list(_SIGS) + ['plaidml_string_ptr', 'plaidml_string_free', 'plaidml_hip_last_run_stats',
                               'plaidml_hip_last_run_memory', 'plaidml_hip_last_run_step_ms', 'plaidml_hip_last_run_replayed',
                               'plaidml_hip_last_run_graph_note'])

_lib = None


def lib():
    """The loaded library.  Raises if it was not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError('%s is missing: build the host library first' % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        for name, (res, args) in _SIGS.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = [ctypes.POINTER(Error)] + args
        L.plaidml_string_ptr.restype = ctypes.c_char_p
        L.plaidml_string_ptr.argtypes = [vp]
        L.plaidml_string_free.restype = None
        L.plaidml_string_free.argtypes = [vp]
        L.plaidml_hip_last_run_stats.restype = None
        L.plaidml_hip_last_run_stats.argtypes = [ctypes.POINTER(f64), ctypes.POINTER(f64), ctypes.POINTER(f64), ctypes.POINTER(sz)]
        L.plaidml_hip_last_run_memory.restype = None
        L.plaidml_hip_last_run_memory.argtypes = [ctypes.POINTER(sz), ctypes.POINTER(sz), ctypes.POINTER(sz)]
        L.plaidml_hip_last_run_step_ms.restype = sz
        L.plaidml_hip_last_run_replayed.restype = ctypes.c_int
        L.plaidml_hip_last_run_replayed.argtypes = []
        L.plaidml_hip_last_run_graph_note.restype = ctypes.c_char_p
        L.plaidml_hip_last_run_graph_note.argtypes = []
        L.plaidml_hip_last_run_step_ms.argtypes = [sz, ctypes.POINTER(f64)]
        _lib = L
        call('plaidml_init')
        call('plaidml_edsl_init')
    return _lib


class PlaidMLError(Exception):
    pass


def call(name, *args):
    """Invokes a C ABI function with a fresh plaidml_error and raises on failure."""
    fn = getattr(_lib if _lib is not None else lib(), name)
    err = Error(0, None)
    ret = fn(ctypes.byref(err), *args)
    if err.code:
        msg = _lib.plaidml_string_ptr(err.msg).decode()
        _lib.plaidml_string_free(err.msg)
        raise PlaidMLError(msg)
    return ret


def _take_str(ptr):
    s = lib().plaidml_string_ptr(ptr).decode()
    _lib.plaidml_string_free(ptr)
    return s


def _ptr_array(ptrs):
    arr = (vp * builtins.max(1, len(ptrs)))()
    for i, p in enumerate(ptrs):
        arr[i] = p
    return arr


class _Handle:
    """Owns one C handle and frees it with the matching *_free."""
    _free = None

    def __init__(self, ptr):
        if not ptr:
            raise PlaidMLError('null handle')
        self._ptr = ptr

    def as_ptr(self):
        return self._ptr

    def __del__(self):
        try:
            if self._ptr and _lib is not None:
                err = Error(0, None)
                getattr(_lib, self._free)(ctypes.byref(err), self._ptr)
                self._ptr = None
        except Exception:
            pass


class DType(enum.IntEnum):
    """plaidml_datatype (plaidml/core/ffi.h:139-156); BFLOAT16 is appended."""
    INVALID = 0
    INTX = 1
    UINTX = 2
    FLOATX = 3
    BOOLEAN = 4
    INT8 = 5
    UINT8 = 6
    INT16 = 7
    UINT16 = 8
    INT32 = 9
    UINT32 = 10
    INT64 = 11
    UINT64 = 12
    FLOAT16 = 13
    FLOAT32 = 14
    FLOAT64 = 15
    BFLOAT16 = 16

    def into_numpy(self):
        return _NUMPY[self]

    @staticmethod
    def from_numpy(dt):
        dt = np.dtype(dt)
        for k, v in _NUMPY.items():
            if k != DType.BFLOAT16 and np.dtype(v) == dt:
                return k
        raise ValueError('unsupported numpy dtype %s' % dt)


_NUMPY = {DType.BOOLEAN: np.bool_, DType.INT8: np.int8, DType.UINT8: np.uint8, DType.INT16: np.int16,
          DType.UINT16: np.uint16, DType.INT32: np.int32, DType.UINT32: np.uint32, DType.INT64: np.int64,
          DType.UINT64: np.uint64, DType.FLOAT16: np.float16, DType.FLOAT32: np.float32, DType.FLOAT64: np.float64,
          DType.BFLOAT16: np.uint16}  # bfloat16 travels as its 16 storage bits


class TensorShape(_Handle):
    _free = 'plaidml_shape_free'

    def __init__(self, dtype=None, sizes=(), strides=None, ptr=None):
        if ptr is None:
            sizes = [int(s) for s in sizes]
            arr = (i64 * builtins.max(1, len(sizes)))(*sizes)
            st = None
            if strides:
                st = (i64 * len(strides))(*[int(s) for s in strides])
            ptr = call('plaidml_shape_alloc', int(dtype), len(sizes), arr, st)
        super().__init__(ptr)

    def _ints(self, fn):
        p = call(fn, self._ptr)
        out = [int(p.contents.elts[i]) for i in range(p.contents.size)]
        call('plaidml_integers_free', ctypes.cast(p, vp))
        return out

    @property
    def dtype(self):
        return DType(call('plaidml_shape_get_dtype', self._ptr))

    @property
    def rank(self):
        return call('plaidml_shape_get_rank', self._ptr)

    @property
    def sizes(self):
        return self._ints('plaidml_shape_get_sizes')

    @property
    def strides(self):
        return self._ints('plaidml_shape_get_strides')

    def byte_size(self):
        return call('plaidml_shape_get_nbytes', self._ptr)

    def __str__(self):
        return _take_str(call('plaidml_shape_repr', self._ptr))


class Buffer(_Handle):
    """Host memory.  Buffer(shape) allocates zero-filled memory; Buffer(shape, data=ndarray) adopts the array."""
    _free = 'plaidml_buffer_free'

    def __init__(self, shape=None, ptr=None, data=None):
        self._keep = None
        if ptr is None:
            if data is not None:
                data = np.ascontiguousarray(data)
                self._keep = data
                ptr = call('plaidml_buffer_adopt', shape.as_ptr(), data.ctypes.data, data.nbytes)
            else:
                ptr = call('plaidml_buffer_alloc', shape.as_ptr())
        super().__init__(ptr)

    @property
    def shape(self):
        return TensorShape(ptr=call('plaidml_buffer_shape', self._ptr))

    def size(self):
        return call('plaidml_buffer_size', self._ptr)

    def as_ndarray(self):
        shape = self.shape
        n = self.size()
        raw = (ctypes.c_char * n).from_address(call('plaidml_buffer_data', self._ptr))
        return np.frombuffer(raw, dtype=shape.dtype.into_numpy()).reshape(shape.sizes).copy()

    def copy_from_ndarray(self, src):
        src = np.ascontiguousarray(src, dtype=self.shape.dtype.into_numpy())
        if src.nbytes != self.size():
            raise ValueError('size mismatch in copy_from_ndarray')
        ctypes.memmove(call('plaidml_buffer_data', self._ptr), src.ctypes.data, src.nbytes)


# ---- dims and index polynomials ------------------------------------------------------------------

_INT_OP = {'neg': 0, 'add': 1, 'sub': 2, 'mul': 3, 'div': 4, 'max': 5, 'min': 6}


def _wrap_dim(x):
    return x if isinstance(x, TensorDim) else TensorDim(int(x))


class TensorDim(_Handle):
    _free = 'plaidml_dim_expr_free'

    def __init__(self, value=None, ptr=None):
        if ptr is None:
            ptr = call('plaidml_dim_expr_none') if value is None else call('plaidml_dim_expr_int', int(value))
        super().__init__(ptr)

    @staticmethod
    def _op(op, *args):
        args = [_wrap_dim(a) for a in args]
        return TensorDim(ptr=call('plaidml_dim_expr_op', _INT_OP[op], len(args), _ptr_array([a.as_ptr() for a in args])))

    def __neg__(self):
        return TensorDim._op('neg', self)

    def __add__(self, o):
        return TensorDim._op('add', self, o)

    def __radd__(self, o):
        return TensorDim._op('add', o, self)

    def __sub__(self, o):
        return TensorDim._op('sub', self, o)

    def __rsub__(self, o):
        return TensorDim._op('sub', o, self)

    def __mul__(self, o):
        return TensorDim._op('mul', self, o)

    def __rmul__(self, o):
        return TensorDim._op('mul', o, self)

    def __floordiv__(self, o):
        return TensorDim._op('div', self, o)

    def __rfloordiv__(self, o):
        return TensorDim._op('div', o, self)

    def __str__(self):
        return _take_str(call('plaidml_dim_expr_repr', self._ptr))


def TensorDims(count):
    return [TensorDim() for _ in range(count)]


def _wrap_poly(x):
    if isinstance(x, TensorIndex):
        return x
    if isinstance(x, TensorDim):
        return TensorIndex(ptr=call('plaidml_poly_expr_dim', x.as_ptr()))
    return TensorIndex(ptr=call('plaidml_poly_expr_literal', int(x)))


class Constraint:
    def __init__(self, lhs, rhs):
        self.lhs, self.rhs = lhs, _wrap_dim(rhs)


class TensorIndex(_Handle):
    _free = 'plaidml_poly_expr_free'

    def __init__(self, name='', ptr=None):
        if ptr is None:
            ptr = call('plaidml_poly_expr_index', name.encode())
        super().__init__(ptr)

    @staticmethod
    def _op(op, *args):
        args = [_wrap_poly(a) for a in args]
        return TensorIndex(ptr=call('plaidml_poly_expr_op', _INT_OP[op], len(args), _ptr_array([a.as_ptr() for a in args])))

    def __lt__(self, rhs):
        return Constraint(self, rhs)

    def __neg__(self):
        return TensorIndex._op('neg', self)

    def __add__(self, o):
        return TensorIndex._op('add', self, o)

    def __radd__(self, o):
        return TensorIndex._op('add', o, self)

    def __sub__(self, o):
        return TensorIndex._op('sub', self, o)

    def __rsub__(self, o):
        return TensorIndex._op('sub', o, self)

    def __mul__(self, o):
        return TensorIndex._op('mul', self, o)

    def __rmul__(self, o):
        return TensorIndex._op('mul', o, self)

    def __floordiv__(self, o):
        return TensorIndex._op('div', self, o)

    def __str__(self):
        return _take_str(call('plaidml_poly_expr_repr', self._ptr))


def TensorIndexes(count):
    return [TensorIndex() for _ in range(count)]


# ---- tensors -----------------------------------------------------------------------------------------

_AGG = {'sum': 1, 'max': 2, 'min': 3, 'product': 4, 'assign': 5}
_COMBO = {'none': 0, 'mul': 1, 'add': 2, 'eq': 3, 'cond': 4}


class IndexedTensor:
    def __init__(self, op, ref=None, idxs=None, args=None):
        self._op, self._ref, self._idxs, self._args = op, ref, idxs, args

    def __add__(self, rhs):
        return IndexedTensor('add', args=[self, rhs])

    def __mul__(self, rhs):
        return IndexedTensor('mul', args=[self, rhs])

    def __eq__(self, rhs):
        return IndexedTensor('eq', args=[self, rhs])

    __hash__ = object.__hash__


def cond(lhs, rhs, true_case):
    return IndexedTensor('cond', args=[lhs, rhs, true_case])


def _wrap_tensor(x):
    if isinstance(x, Tensor):
        return x
    if isinstance(x, TensorDim):
        return Tensor(ptr=call('plaidml_expr_dim', x.as_ptr()))
    if isinstance(x, (bool, np.bool_)):
        return Tensor(ptr=call('plaidml_expr_int', int(x)))
    if isinstance(x, (int, np.integer)):
        return Tensor(ptr=call('plaidml_expr_int', int(x)))
    if isinstance(x, (float, np.floating)):
        return Tensor(ptr=call('plaidml_expr_float', float(x)))
    raise TypeError('cannot convert %r to a Tensor' % (x,))


def intrinsic(fn, *args, name=''):
    args = [_wrap_tensor(a) for a in args]
    return Tensor(ptr=call('plaidml_expr_intrinsic', fn.encode(), len(args), _ptr_array([a.as_ptr() for a in args]), name.encode()))


class Tensor(_Handle):
    _free = 'plaidml_expr_free'

    def __init__(self, ptr=None, value=None):
        self._buffer = None
        if ptr is None:
            ptr = _wrap_tensor(value)._steal()
        super().__init__(ptr)

    def _steal(self):
        p, self._ptr = self._ptr, None
        return p

    _lens = None  # a TensorLens set by use(): dimensions and indexes are then given in the lens's source order

    def use(self, lens):
        """The same tensor seen through `lens` (plaidml/edsl/__init__.py:645-646)."""
        t = Tensor(ptr=call('plaidml_expr_clone', self._ptr))
        t._lens = lens
        return t

    def __getitem__(self, key):
        if not isinstance(key, (tuple, list)):
            key = (key,)
        key = list(key) if self._lens is None else self._lens.apply(list(key))
        return IndexedTensor('none', ref=self, idxs=[_wrap_poly(k) for k in key])

    def __neg__(self):
        return intrinsic('neg', self)

    def __add__(self, r):
        return intrinsic('add', self, r)

    def __radd__(self, l):
        return intrinsic('add', l, self)

    def __sub__(self, r):
        return intrinsic('sub', self, r)

    def __rsub__(self, l):
        return intrinsic('sub', l, self)

    def __mul__(self, r):
        return intrinsic('mul', self, r)

    def __rmul__(self, l):
        return intrinsic('mul', l, self)

    def __truediv__(self, r):
        return intrinsic('div', self, r)

    def __rtruediv__(self, l):
        return intrinsic('div', l, self)

    def __eq__(self, r):
        return intrinsic('cmp_eq', self, r)

    def __ne__(self, r):
        return intrinsic('cmp_ne', self, r)

    def __lt__(self, r):
        return intrinsic('cmp_lt', self, r)

    def __gt__(self, r):
        return intrinsic('cmp_gt', self, r)

    def __le__(self, r):
        return intrinsic('cmp_le', self, r)

    def __ge__(self, r):
        return intrinsic('cmp_ge', self, r)

    def __mod__(self, r):
        return intrinsic('mod', self, r)

    def __rmod__(self, l):
        return intrinsic('mod', l, self)

    def __and__(self, r):
        return intrinsic('bit_and', self, r)

    def __rand__(self, l):
        return intrinsic('bit_and', l, self)

    def __or__(self, r):
        return intrinsic('bit_or', self, r)

    def __ror__(self, l):
        return intrinsic('bit_or', l, self)

    def __xor__(self, r):
        return intrinsic('bit_xor', self, r)

    def __rxor__(self, l):
        return intrinsic('bit_xor', l, self)

    def __lshift__(self, r):
        return intrinsic('bit_shl', self, r)

    def __rlshift__(self, l):
        return intrinsic('bit_shl', l, self)

    def __rshift__(self, r):
        return intrinsic('bit_shr', self, r)

    def __rrshift__(self, l):
        return intrinsic('bit_shr', l, self)

    def __invert__(self):
        return intrinsic('bit_not', self)

    __hash__ = object.__hash__

    def compute_shape(self):
        return TensorShape(ptr=call('plaidml_expr_get_shape', self._ptr))

    @property
    def shape(self):
        return tuple(self.compute_shape().sizes)

    @property
    def dtype(self):
        return DType(call('plaidml_expr_get_dtype', self._ptr))

    dt = dtype

    @property
    def rank(self):
        return call('plaidml_expr_get_rank', self._ptr)

    def bind_dims(self, *dims):
        if len(dims) == 1 and isinstance(dims[0], (list, tuple)):
            dims = dims[0]
        dims = list(dims) if self._lens is None else self._lens.apply(list(dims))
        call('plaidml_expr_bind_dims', self._ptr, len(dims), _ptr_array([d.as_ptr() for d in dims]))

    def __str__(self):
        return _take_str(call('plaidml_expr_repr', self._ptr))


class TensorLens:
    """A change of dimension order: position i of what the user writes (in `source` order) lands where the
    letter source[i] stands in `target` (plaidml/edsl/__init__.py:292-309)."""

    def __init__(self, source='', target=''):
        if len(source) != len(target):
            raise ValueError('source and target rank mismatch')
        self.map = []
        for ch in source:
            pos = target.find(ch)
            if pos == -1:
                raise ValueError('source and target dims mismatch')
            self.map.append(pos)

    def apply(self, items):
        if not self.map:
            return items
        if len(items) != len(self.map):
            raise ValueError('rank mismatch in TensorLens apply')
        return [items[x] for x in self.map]


class Contraction:
    def __init__(self, lens=None, name=''):
        if isinstance(lens, str):  # Contraction('name')
            lens, name = None, lens
        self._lens = lens
        self._name = name
        self._dims, self._idxs, self._agg, self._rhs, self._init, self._cons = [], [], None, None, None, []

    def outShape(self, *args):
        if len(args) == 1 and isinstance(args[0], (list, tuple)):
            args = args[0]
        self._dims = [_wrap_dim(a) for a in args]
        return self

    def outAccess(self, *args):
        if len(args) == 1 and isinstance(args[0], (list, tuple)):
            args = args[0]
        self._idxs = [_wrap_poly(a) for a in args]
        return self

    def _set(self, agg, rhs):
        self._agg, self._rhs = agg, rhs
        return self

    def assign(self, rhs):
        return self._set('assign', rhs)

    def max(self, rhs):
        return self._set('max', rhs)

    def min(self, rhs):
        return self._set('min', rhs)

    def product(self, rhs):
        return self._set('product', rhs)

    def sum(self, rhs):
        return self._set('sum', rhs)

    def init(self, rhs):
        self._init = rhs
        return self

    def add_constraint(self, c):
        self._cons.append(c)
        return self

    def add_constraints(self, cs):
        self._cons.extend(cs)
        return self

    def build(self):
        rhs = self._rhs
        if isinstance(rhs, Tensor):
            rhs = IndexedTensor('none', ref=rhs, idxs=[])
        idxs = self._idxs if self._lens is None else self._lens.apply(self._idxs)
        dims = self._dims if self._lens is None else self._lens.apply(self._dims)
        t = Tensor(ptr=call('plaidml_expr_contraction', _AGG[self._agg], _COMBO[rhs._op], len(idxs),
                            _ptr_array([i.as_ptr() for i in idxs]), _ptr_array([d.as_ptr() for d in dims]),
                            self._init.as_ptr() if self._init is not None else None, self._name.encode()))
        operands = [rhs] if rhs._op == 'none' else rhs._args
        for o in operands:
            call('plaidml_contraction_add_operand', t.as_ptr(), o._ref.as_ptr(), len(o._idxs),
                 _ptr_array([i.as_ptr() for i in o._idxs]))
        for c in self._cons:
            call('plaidml_contraction_add_constraint', t.as_ptr(), c.lhs.as_ptr(), c.rhs.as_ptr())
        call('plaidml_contraction_build', t.as_ptr())
        return t


def Placeholder(dtype_or_shape, dims=(), name=''):
    shape = dtype_or_shape if isinstance(dtype_or_shape, TensorShape) else TensorShape(dtype_or_shape, dims)
    return Tensor(ptr=call('plaidml_expr_input', shape.as_ptr(), name.encode()))


def Constant(value, dtype=None, name=''):
    """A tensor constant from a numpy array (dtype=DType.BFLOAT16 with a uint16 array of storage bits,
    or with a float32 array that is rounded), or a scalar literal."""
    if isinstance(value, np.ndarray):
        dt = DType(dtype) if dtype is not None else DType.from_numpy(value.dtype)
        if dt == DType.BFLOAT16 and value.dtype != np.uint16:
            value = to_bf16_bits(value)
        value = np.ascontiguousarray(value, dtype=dt.into_numpy())
        # copied into library-owned memory: the expression graph outlives the numpy array
        buf = Buffer(TensorShape(dt, value.shape))
        buf.copy_from_ndarray(value)
        return Tensor(ptr=call('plaidml_expr_constant', buf.as_ptr(), name.encode()))
    return _wrap_tensor(value)


def cast(x, dtype):
    x = _wrap_tensor(x)  # must stay alive across the call
    return Tensor(ptr=call('plaidml_expr_cast', x.as_ptr(), int(dtype)))


def index(dims, axis):
    return intrinsic('index', int(axis), *[_wrap_dim(d) for d in dims])


def reshape(x, dims):
    return intrinsic('reshape', x, *[_wrap_dim(d) for d in dims])


def select(c, t, f):
    return intrinsic('select', c, t, f)


def _unary(fn):
    def f(x):
        return intrinsic(fn, x)
    f.__name__ = fn
    return f


ceil, exp, floor, ident, log, relu, sqrt, tanh = (_unary(n) for n in ('ceil', 'exp', 'floor', 'ident', 'log', 'relu', 'sqrt', 'tanh'))
round = _unary('round')  # noqa: A001
sin, cos, tan, sinh, cosh, asin, acos, atan, asinh, acosh, atanh, erf = (
    _unary(n) for n in ('sin', 'cos', 'tan', 'sinh', 'cosh', 'asin', 'acos', 'atan', 'asinh', 'acosh', 'atanh', 'erf'))
logical_not = _unary('logical_not')
shape_of = _unary('shape')   # the extents of a tensor as an si32 vector (edsl `shape`)


def pow(x, y):  # noqa: A001
    return intrinsic('pow', x, y)


def logical_and(x, y):
    return intrinsic('logical_and', x, y)


def logical_or(x, y):
    return intrinsic('logical_or', x, y)


def logical_xor(x, y):
    return intrinsic('logical_xor', x, y)


def max(x, y):  # noqa: A001
    return select(_wrap_tensor(x) < y, y, x)


def min(x, y):  # noqa: A001
    return select(_wrap_tensor(x) < y, x, y)


def abs(x):  # noqa: A001
    return select(x < 0.0, -x, x)


# ---- special operations (plaidml/edsl/edsl.h:800-811, 1034-1066, 1625-1765) ----------------------------------
SORT_ASC, SORT_DESC = range(2)
INTERP_NEAREST, INTERP_LINEAR, INTERP_CUBIC, INTERP_NONE = range(4)
NEAREST_ROUND_PREFER_FLOOR, NEAREST_ROUND_PREFER_CEIL, NEAREST_FLOOR, NEAREST_CEIL, NEAREST_SIMPLE, NEAREST_NONE = range(6)
GATHER_NORMAL, GATHER_ND = range(2)
OOB_EDGE_PADDED_INPUT, OOB_RETURN_ZERO = range(2)
SCATTER_NORMAL, SCATTER_UPDATE_SLICE, SCATTER_UPDATE_ELT, SCATTER_UPDATE_ND = range(4)


def _const(ptr):
    return Tensor(ptr=ptr)


def _uint(v):
    return _const(call('plaidml_expr_uint', int(v)))


def _int(v):
    return _const(call('plaidml_expr_int', int(v)))


def _float(v):
    return _const(call('plaidml_expr_float', float(v)))


def prng(state, dims):
    """(values of shape dims in [0, 1), advanced state): plaidml/edsl/edsl.h:971-979."""
    r = intrinsic('prng', state, *[TensorDim(int(d)) for d in dims])
    return (Tensor(ptr=call('plaidml_expr_element', r.as_ptr(), 0)), Tensor(ptr=call('plaidml_expr_element', r.as_ptr(), 1)))


def argsort(x, axis=-1, direction=SORT_ASC):
    return intrinsic('argsort', x, _int(axis), _int(direction))


def gather(x, y, axis=0, interpolation_mode=INTERP_NONE, nearest_mode=NEAREST_ROUND_PREFER_FLOOR, cube_coeff=-0.75,
           mode=GATHER_NORMAL, batch_dims=0, out_of_bounds_mode=OOB_EDGE_PADDED_INPUT):
    # a plain number addresses one position and keeps the axis, as the C++ builder's scalar overloads do
    # (plaidml/edsl/edsl.h:1699-1717)
    if isinstance(y, bool):
        raise TypeError('gather index must be a tensor or a number')
    if isinstance(y, int):
        y = cast(index([1], 0), DType.INT32) + y
    elif isinstance(y, float):
        y = cast(index([1], 0), DType.FLOAT32) + y
    if axis < 0:
        axis += x.rank
    return intrinsic('gather', x, y, _uint(axis), _uint(interpolation_mode), _uint(nearest_mode), _float(cube_coeff), _uint(mode),
                     _uint(batch_dims), _uint(out_of_bounds_mode))


def trace(x, msg):
    """A trace marker passes its tensor through (the reference prints `msg` when the value is computed)."""
    return x


def scatter(x, y, z, axis=0, mode=SCATTER_NORMAL):
    if axis < 0:
        axis += x.rank
    return intrinsic('scatter', x, y, z, _int(axis), _uint(mode))


# ---- values (arguments of the operation library) ------------------------------------------------------

class Value(_Handle):
    _free = 'plaidml_value_free'

    def __init__(self, value=None, ptr=None):
        if ptr is None:
            if value is None:
                ptr = call('plaidml_value_none')
            elif isinstance(value, Value):
                ptr = call('plaidml_value_clone', value.as_ptr())
            elif isinstance(value, Tensor):
                ptr = call('plaidml_value_expr', value.as_ptr())
            elif isinstance(value, TensorDim):
                ptr = call('plaidml_value_dim', value.as_ptr())
            elif isinstance(value, (bool, np.bool_, int, np.integer)):
                ptr = call('plaidml_value_int', int(value))
            elif isinstance(value, (float, np.floating)):
                ptr = call('plaidml_value_float', float(value))
            elif isinstance(value, str):
                ptr = call('plaidml_value_str', value.encode())
            elif isinstance(value, (list, tuple)):
                elts = [Value(v) for v in value]
                ptr = call('plaidml_value_tuple', len(elts), _ptr_array([e.as_ptr() for e in elts]))
            else:
                raise TypeError('unsupported Value %r' % (value,))
        super().__init__(ptr)

    def as_tensor(self):
        return Tensor(ptr=call('plaidml_value_expr_get', self._ptr))

    def as_tuple(self):
        # the elements become this caller's handles; plaidml_tuple_free releases the container only
        lst = call('plaidml_value_tuple_get', self._ptr)
        try:
            return [Value(ptr=lst.contents.elts[i]) for i in range(lst.contents.size)]
        finally:
            call('plaidml_tuple_free', lst)

    def __str__(self):
        return _take_str(call('plaidml_value_repr', self._ptr))


def op_make(name, args):
    packed = Value(args)  # must stay alive across the call
    return Value(ptr=call('plaidml_op_make', name.encode(), packed.as_ptr()))


# ---- programs and execution --------------------------------------------------------------------------

def list_targets():
    p = call('plaidml_targets_get')
    out = [_take_str(p.contents.elts[i]) for i in range(p.contents.size)]
    call('plaidml_strings_free', ctypes.cast(p, vp))
    return out


def list_devices():
    call('plaidml_exec_init')
    p = call('plaidml_devices_get')
    out = [_take_str(p.contents.elts[i]) for i in range(p.contents.size)]
    call('plaidml_strings_free', ctypes.cast(p, vp))
    return out


class Program(_Handle):
    _free = 'plaidml_program_free'

    def __init__(self, name, inputs, outputs):
        self._inputs, self._outputs = list(inputs), list(outputs)  # keep expressions (and adopted constants) alive
        ptr = call('plaidml_build', name.encode(), len(inputs), _ptr_array([t.as_ptr() for t in inputs]), None, len(outputs),
                   _ptr_array([t.as_ptr() for t in outputs]))
        super().__init__(ptr)

    def compile(self, target='', debug=False):
        call('plaidml_program_compile', self._ptr, debug, target.encode())

    def _shapes(self, fn):
        p = call(fn, self._ptr)
        out = [TensorShape(ptr=p.contents.elts[i]) for i in range(p.contents.size)]
        call('plaidml_shapes_free', ctypes.cast(p, vp))
        return out

    @property
    def inputs(self):
        return self._shapes('plaidml_program_get_inputs')

    @property
    def outputs(self):
        return self._shapes('plaidml_program_get_outputs')

    @property
    def passes(self):
        p = call('plaidml_program_get_passes', self._ptr)
        out = [(_take_str(p.contents.elts[i].key), _take_str(p.contents.elts[i].value)) for i in range(p.contents.size)]
        call('plaidml_kvps_free', ctypes.cast(p, vp))
        return out

    def __str__(self):
        return _take_str(call('plaidml_program_repr', self._ptr))


class Executable(_Handle):
    _free = 'plaidml_executable_free'

    def __init__(self, program, device=''):
        call('plaidml_exec_init')
        self._program = program
        super().__init__(call('plaidml_jit', program.as_ptr(), device.encode()))

    def run(self, inputs, outputs):
        """inputs / outputs: lists of Buffer.  Returns the wall time of the run in ms, transfers included."""
        return call('plaidml_executable_run', self._ptr, len(inputs), _ptr_array([b.as_ptr() for b in inputs]), len(outputs),
                    _ptr_array([b.as_ptr() for b in outputs]))


def last_run_stats():
    k, h, d, n = f64(), f64(), f64(), sz()
    lib().plaidml_hip_last_run_stats(ctypes.byref(k), ctypes.byref(h), ctypes.byref(d), ctypes.byref(n))
    a, u, t = sz(), sz(), sz()
    lib().plaidml_hip_last_run_memory(ctypes.byref(a), ctypes.byref(u), ctypes.byref(t))
    steps = (f64 * (n.value or 1))()
    got = lib().plaidml_hip_last_run_step_ms(n.value, steps)  # per launch; empty unless PLAIDML_PROFILE=1 was set
    return {'kernel_ms': k.value, 'h2d_ms': h.value, 'd2h_ms': d.value, 'launches': n.value, 'arena_bytes': a.value,
            'unshared_temp_bytes': u.value, 'device_bytes': t.value, 'graph': bool(lib().plaidml_hip_last_run_replayed()),
            'graph_note': lib().plaidml_hip_last_run_graph_note().decode(), 'step_ms': [steps[i] for i in range(got if got < n.value else n.value)]}


def to_bf16_bits(a):
    """float32 -> bfloat16 storage bits, round to nearest even."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    bits = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    bits[np.isnan(a)] = 0x7FC0
    return bits


def from_bf16_bits(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def round_bf16(a):
    """float32 -> the nearest bfloat16 value (ties to even), as float32."""
    return from_bf16_bits(to_bf16_bits(a))


class Runner:
    """Compiles once, then runs with numpy arrays (reference: plaidml/exec/__init__.py:49-63).
    bfloat16 inputs are given as float32 arrays (rounded on the way in) and returned as float32."""

    def __init__(self, program, device='', target=''):
        program.compile(target)
        self.program = program
        self.exe = Executable(program, device)
        self.in_shapes = program.inputs
        self.out_shapes = program.outputs
        self.outputs = [Buffer(s) for s in self.out_shapes]

    def _converted(self, inputs):
        for shape, a in zip(self.in_shapes, inputs):
            dt = shape.dtype
            a = np.asarray(a)
            if dt == DType.BFLOAT16 and a.dtype != np.uint16:
                a = to_bf16_bits(a)
            yield shape, np.ascontiguousarray(a, dtype=dt.into_numpy()).reshape(shape.sizes)

    def stage(self, inputs):
        """Converts the inputs once into buffers of the library's own (page-locked where large) memory, for
        callers that run the same batch many times; returns the list to pass to run_staged."""
        bufs = []
        for shape, a in self._converted(inputs):
            b = Buffer(shape)
            b.copy_from_ndarray(a)
            bufs.append(b)
        return bufs

    def run_staged(self, bufs):
        """One run over staged inputs; results stay in self.outputs until fetch().  Returns the wall ms."""
        self.ms = self.exe.run(bufs, self.outputs)
        return self.ms

    def run(self, inputs):
        self.ms = self.exe.run([Buffer(shape, data=a) for shape, a in self._converted(inputs)], self.outputs)
        return self.fetch()

    def fetch(self):
        outs = []
        for shape, b in zip(self.out_shapes, self.outputs):
            a = b.as_ndarray()
            outs.append(from_bf16_bits(a) if shape.dtype == DType.BFLOAT16 else a)
        return outs


def run(program, inputs, device='', target=''):
    return Runner(program, device, target).run(inputs)

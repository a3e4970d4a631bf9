"""TEST INFRASTRUCTURE -- ctypes door onto liboracle_kernels.so (oracle/kernels.c).

Views are numpy arrays plus a layout permutation; `View` builds the same
(shape, element strides) description the product's C ABI takes, but over host
memory.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

FL_MAX_RANK = 8
FL_BOOL, FL_INT32, FL_INT64, FL_FLOAT16, FL_FLOAT32, FL_FLOAT64 = 1, 2, 3, 4, 5, 6
NP_TO_FL = {
    np.dtype(np.bool_): FL_BOOL,
    np.dtype(np.uint8): FL_BOOL,
    np.dtype(np.int32): FL_INT32,
    np.dtype(np.int64): FL_INT64,
    np.dtype(np.float32): FL_FLOAT32,
    np.dtype(np.float64): FL_FLOAT64,
}

# op codes of kernels.c
OP_ADD_C, OP_RSUB_C, OP_MUL_C, OP_DIV_C, OP_POW_C, OP_ERF, OP_RELU, OP_CLIP, OP_TANH, OP_SQRT, OP_NEG, OP_COPY = range(12)
IOP_ADD_C, IOP_CAST, IOP_EQ_C, IOP_NOT = range(4)
BOP_ADD, BOP_SUB, BOP_MUL, BOP_DIV = range(4)


class CView(ctypes.Structure):
    _fields_ = [
        ("base", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("rank", ctypes.c_int32),
        ("shape", ctypes.c_int64 * FL_MAX_RANK),
        ("strides", ctypes.c_int64 * FL_MAX_RANK),
    ]


_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle_kernels.so")
if not os.path.exists(LIB_PATH):
    raise ImportError(f"{LIB_PATH} missing: run `make -C oracle kernels`")
lib = ctypes.CDLL(LIB_PATH)


def physical_shape(shape, layout):
    phys = [0] * len(shape)
    for i, j in enumerate(layout):
        phys[j] = int(shape[i])
    return phys


def row_major_strides(shape):
    strides = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        strides[i - 1] = strides[i] * int(shape[i])
    return strides


def layout_strides(shape, layout):
    phys = row_major_strides(physical_shape(shape, layout))
    return [phys[j] for j in layout]


def reference_constant(logical: np.ndarray, layout):
    """A constant tensor as the reference stores it and as its kernels then read it, for a layout other than the
    default one (reference src/worker/builder.cpp:279-297 for float32, :306-318 for int64): the global's dense data
    is written in row-major order of the logical indices, entry n taking buffer[GenIndex(indices_n, strides)], and the
    kernels address the global through those same strides.  Returns (data as stored, tensor as read)."""
    logical = np.asarray(logical)
    shape = list(logical.shape)
    strides = np.asarray(layout_strides(shape, layout), dtype=np.int64)
    indices = np.indices(shape).reshape(len(shape), -1)  # column n = the n-th index tuple in row-major order
    strided = (indices * strides[:, None]).sum(axis=0)
    stored = logical.reshape(-1)[strided]
    return stored, stored[strided].reshape(shape)


class View:
    """A logical tensor stored in host memory with a layout permutation
    (layout[i] = physical position of logical dim i)."""

    def __init__(self, logical: np.ndarray, layout=None):
        logical = np.asarray(logical)
        rank = logical.ndim
        self.layout = list(range(rank)) if layout is None else [int(v) for v in layout]
        self.shape = list(logical.shape)
        inv = [0] * rank
        for i, j in enumerate(self.layout):
            inv[j] = i
        # physical array P with P.transpose(layout) == logical
        self.physical = np.ascontiguousarray(np.transpose(logical, inv)) if rank else np.array(logical)
        self.strides = layout_strides(self.shape, self.layout) if rank else []
        self.dtype = NP_TO_FL[self.physical.dtype]

    @classmethod
    def empty(cls, shape, dtype=np.float32, layout=None, fill=0):
        return cls(np.full(shape, fill, dtype=dtype), layout)

    def logical(self) -> np.ndarray:
        return np.transpose(self.physical, self.layout) if self.shape else self.physical

    def c(self) -> CView:
        v = CView()
        v.base = self.physical.ctypes.data
        v.dtype = self.dtype
        v.rank = len(self.shape)
        for i, (s, st) in enumerate(zip(self.shape, self.strides)):
            v.shape[i] = s
            v.strides[i] = st
        return v


def _ref(v):
    return None if v is None else ctypes.byref(v.c())


def _i64(values):
    vals = [int(v) for v in values]
    return (ctypes.c_int64 * max(1, len(vals)))(*vals)


def _call(name, *args):
    fn = getattr(lib, name)
    fn.restype = ctypes.c_int
    rc = fn(*args)
    if rc != 0:
        raise RuntimeError(f"{name} returned {rc}")


d = ctypes.c_double
i32 = ctypes.c_int32
i64 = ctypes.c_int64
u32 = ctypes.c_uint32


def unary_f32(op, x: View, out: View, c0=0.0, c1=0.0):
    _call("oracle_unary_f32", i32(op), _ref(x), _ref(out), d(c0), d(c1))


def unary_int(op, x: View, out: View, c=0.0):
    _call("oracle_unary_int", i32(op), _ref(x), _ref(out), d(c))


def binary_f32(op, a: View, b: View, out: View):
    _call("oracle_binary_f32", i32(op), _ref(a), _ref(b), _ref(out))


def mul_int(a, b, out):
    _call("oracle_mul_int", _ref(a), _ref(b), _ref(out))


def where(cond, x, y_tensor, y_scalar, out):
    _call("oracle_where", _ref(cond), _ref(x), _ref(y_tensor), d(y_scalar), _ref(out))


def add_div_erf_add_mul_mul(x, add0, out, div, add1, mul1):
    _call("oracle_add_div_erf_add_mul_mul", _ref(x), _ref(add0), _ref(out), d(div), d(add1), d(mul1))


def unsqueeze_sub_mul(x, out, axes, sub, mul):
    _call("oracle_unsqueeze_sub_mul", _ref(x), _ref(out), _i64(axes), i32(len(axes)), d(sub), d(mul))


def transpose(x, out, perm):
    _call("oracle_transpose", _ref(x), _ref(out), _i64(perm))


def reshape(x, out):
    _call("oracle_reshape", _ref(x), _ref(out))


def squeeze(x, out, axes):
    _call("oracle_squeeze", _ref(x), _ref(out), _i64(axes), i32(len(axes)))


def unsqueeze(x, out, axes):
    _call("oracle_unsqueeze", _ref(x), _ref(out), _i64(axes), i32(len(axes)))


def slice_(x, out, starts, axes, steps):
    _call("oracle_slice", _ref(x), _ref(out), _i64(starts), _i64(axes), _i64(steps), i32(len(axes)))


def concat2(a, b, out, axis):
    _call("oracle_concat2", _ref(a), _ref(b), _ref(out), i64(axis))


def pad(x, out, pads_before, flags=0):
    """flags = 0: border written as zero; FL_REF_PAD_BORDER_UNWRITTEN (1 << 5): border left as it is"""
    _call("oracle_pad", _ref(x), _ref(out), _i64(pads_before), u32(flags))


def gather_index_scalar(x, out, axis, index, flags=0):
    _call("oracle_gather_index_scalar", _ref(x), _ref(out), i64(axis), i64(index), u32(flags))


def gather_indices_tensor(x, indices, out, axis):
    _call("oracle_gather_indices_tensor", _ref(x), _ref(indices), _ref(out), i64(axis))


def gather_data_tensor(indices, data, out, add0=None, add1=None):
    _call("oracle_gather_data_tensor", _ref(indices), _ref(data), _ref(add0), _ref(add1), _ref(out))


def cum_sum(x, out, axis):
    _call("oracle_cum_sum", _ref(x), _ref(out), i64(axis))


def softmax(x, out, axis):
    rows = int(np.prod(x.shape)) // x.shape[axis]
    scratch = np.zeros(max(rows, 1), dtype=np.float32)
    _call("oracle_softmax", _ref(x), _ref(out), ctypes.c_void_p(scratch.ctypes.data), i64(axis))


def layer_norm(x, scale, bias, out, axis, eps, scratch=None):
    rows = int(np.prod(x.shape)) // x.shape[axis]
    if scratch is None:
        scratch = np.zeros(max(rows, 1), dtype=np.float32)
    else:
        scratch = np.ascontiguousarray(scratch, dtype=np.float32).copy()
        assert scratch.size >= rows
    _call("oracle_layer_norm", _ref(x), _ref(scale), _ref(bias), _ref(out), ctypes.c_void_p(scratch.ctypes.data),
          i64(axis), d(eps))


def reduce_mean(x, out, axes):
    _call("oracle_reduce_mean", _ref(x), _ref(out), _i64(axes), i32(len(axes)))


def pool(is_max, x, out, kernel_shape, strides):
    _call("oracle_pool", i32(1 if is_max else 0), _ref(x), _ref(out), _i64(kernel_shape), _i64(strides),
          i32(len(kernel_shape)))


def matmul(a, b, out):
    _call("oracle_matmul", _ref(a), _ref(b), _ref(out))


def gemm(a, b, bias, out, alpha, beta, trans_a, trans_b, flags=0):
    _call("oracle_gemm", _ref(a), _ref(b), _ref(bias), _ref(out), d(alpha), d(beta), i32(trans_a), i32(trans_b),
          u32(flags))


def conv(x, w, bias, out, pads, strides, dilations, group, flags=0):
    _call("oracle_conv", _ref(x), _ref(w), _ref(bias), _ref(out), None if pads is None else _i64(pads),
          _i64(strides), _i64(dilations), i64(group), u32(flags))

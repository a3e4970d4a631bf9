"""ctypes binding of the C ABI declared in include/fluidml_hip.h.

This is the thinnest possible Python door onto the gfx950 kernels: it loads
``fluidml_amd/lib/libfluidml_hip.so`` (built by ``fluidml_amd/csrc/Makefile``),
declares every entry point's signature and offers helpers to describe a strided
device tensor the way FluidML's builder describes a memref (shape + element
strides derived from a layout permutation, reference src/utils/utils.cpp:64-102).

There is no CPU fallback: if the library is missing, importing this module
raises, and every non-zero return code becomes a ``FluidmlHipError``.
"""
from __future__ import annotations

import ctypes
import os
from typing import Iterable, Optional, Sequence

FL_MAX_RANK = 8

# enum fl_dtype (numbering of the reference's ``enum class Type``, include/utils/type.h:11-19)
FL_UNKNOWN, FL_BOOL, FL_INT32, FL_INT64, FL_FLOAT16, FL_FLOAT32, FL_FLOAT64 = range(7)

# enum fl_ref_flags
FL_REF_CONV_UNIT_STRIDE = 1 << 0
FL_REF_CONV_BIAS_INDEX1 = 1 << 1
FL_REF_LN_STALE_SCRATCH = 1 << 2
FL_REF_GEMM_SWAPPED_SCALARS = 1 << 3
FL_REF_GATHER_RAW_AXIS = 1 << 4
FL_REF_PAD_BORDER_UNWRITTEN = 1 << 5
FL_REF_CONSTANT_GATHERED = 1 << 6
FL_CONTRACT_BF16 = 1 << 0
FL_CONTRACT_ADDEND_IS_FACTOR = 1 << 1
FL_CONTRACT_SHIFT = 16
FL_ERR_NULL = -1
FL_ERR_UNSUPPORTED = -8
FL_ERR_STATIC_SCRATCH = -9
FL_NO_ALLOC_SCRATCH_BYTES = 2 << 20

DTYPE_SIZE = {FL_BOOL: 1, FL_INT32: 4, FL_INT64: 8, FL_FLOAT16: 2, FL_FLOAT32: 4, FL_FLOAT64: 8}


class FlTensor(ctypes.Structure):
    _fields_ = [
        ("base", ctypes.c_void_p),
        ("dtype", ctypes.c_int32),
        ("rank", ctypes.c_int32),
        ("shape", ctypes.c_int64 * FL_MAX_RANK),
        ("strides", ctypes.c_int64 * FL_MAX_RANK),
    ]


class FluidmlHipError(RuntimeError):
    def __init__(self, code: int, what: str):
        super().__init__(f"{what}: {error_string(code)} (code {code})")
        self.code = code


LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libfluidml_hip.so")
if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is missing: build it with `make -C fluidml_amd/csrc hip` "
        "(or `python -c 'import __graft_entry__ as g; g.build()'`); there is no CPU fallback"
    )
lib = ctypes.CDLL(LIB_PATH)

_P = ctypes.POINTER
_T = _P(FlTensor)
_vp = ctypes.c_void_p
_i64p = _P(ctypes.c_int64)
_i32, _i64, _u32, _f64, _f32, _sz = (
    ctypes.c_int32,
    ctypes.c_int64,
    ctypes.c_uint32,
    ctypes.c_double,
    ctypes.c_float,
    ctypes.c_size_t,
)

# name -> argtypes, in the order of include/fluidml_hip.h
SIGNATURES = {
    "fluidml_hip_abi_version": [],
    "fluidml_hip_device_count": [],
    "fluidml_hip_device_info": [ctypes.c_int, ctypes.c_char_p, _sz, ctypes.c_char_p, _sz, _P(ctypes.c_int), _P(_sz)],
    "fluidml_hip_arena_create": [_sz, _P(_vp)],
    "fluidml_hip_arena_destroy": [_vp],
    "fluidml_hip_arena_zero": [_vp, _sz, _vp],
    "fluidml_hip_upload_constant": [_vp, _sz, _P(_vp)],
    "fluidml_hip_free": [_vp],
    "fluidml_hip_memcpy_h2d": [_vp, _vp, _sz, _vp],
    "fluidml_hip_memcpy_d2h": [_vp, _vp, _sz, _vp],
    "fluidml_hip_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "fluidml_hip_time_kernels": [_vp, _vp],
    "fluidml_hip_mfma_rate": [ctypes.c_int32, ctypes.c_int32, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)],
    "fluidml_hip_stream_create": [_P(_vp)],
    "fluidml_hip_stream_destroy": [_vp],
    "fluidml_hip_stream_synchronize": [_vp],
    "fluidml_hip_event_create": [_P(_vp)],
    "fluidml_hip_event_destroy": [_vp],
    "fluidml_hip_event_record": [_vp, _vp],
    "fluidml_hip_stream_wait_event": [_vp, _vp],
    "fluidml_hip_event_elapsed_ns": [_vp, _vp, _P(_f64)],
    "fluidml_hip_graph_begin_capture": [_vp],
    "fluidml_hip_graph_end_capture": [_vp, _P(_vp)],
    "fluidml_hip_graph_launch": [_vp, _vp],
    "fluidml_hip_graph_destroy": [_vp],
    # elementwise
    "fluidml_hip_add_constant": [_T, _T, _f64, _vp],
    "fluidml_hip_add_common": [_T, _T, _T, _vp],
    "fluidml_hip_mul_add": [_T, _T, _T, _T, _vp],
    "fluidml_hip_add_add": [_T, _T, _T, _T, _vp],
    "fluidml_hip_rotary": [_T, _T, _T, _T, _i64, _vp],
    "fluidml_hip_rotary_pair": [_T, _T, _T, _T, _T, _T, _i64, _vp],
    "fluidml_hip_sub_constant_lhs": [_T, _T, _f64, _vp],
    "fluidml_hip_sub_common": [_T, _T, _T, _vp],
    "fluidml_hip_mul_constant": [_T, _T, _f64, _vp],
    "fluidml_hip_mul_common": [_T, _T, _T, _vp],
    "fluidml_hip_div_constant_rhs": [_T, _T, _f64, _vp],
    "fluidml_hip_div_common": [_T, _T, _T, _vp],
    "fluidml_hip_pow": [_T, _T, _f64, _vp],
    "fluidml_hip_erf": [_T, _T, _vp],
    "fluidml_hip_relu": [_T, _T, _vp],
    "fluidml_hip_clip": [_T, _T, _f32, _f32, _vp],
    "fluidml_hip_tanh": [_T, _T, _vp],
    "fluidml_hip_sqrt": [_T, _T, _vp],
    "fluidml_hip_neg": [_T, _T, _vp],
    "fluidml_hip_not": [_T, _T, _vp],
    "fluidml_hip_cast": [_T, _T, _vp],
    "fluidml_hip_equal": [_T, _T, _f64, _vp],
    "fluidml_hip_dropout": [_T, _T, _vp],
    "fluidml_hip_where_constant_cond_constant_scalar_y": [_T, _T, _T, _f64, _vp],
    "fluidml_hip_where_constant_cond_constant_tensor_y": [_T, _T, _T, _T, _vp],
    "fluidml_hip_add_div_erf_add_mul_mul": [_T, _T, _T, _f64, _f64, _f64, _vp],
    "fluidml_hip_unsqueeze_sub_lhs_scalar_mul_rhs_scalar": [_T, _T, _i64p, _i32, _f64, _f64, _vp],
    # data movement
    "fluidml_hip_transpose": [_T, _T, _i64p, _i32, _vp],
    "fluidml_hip_reshape": [_T, _T, _vp],
    "fluidml_hip_flatten": [_T, _T, _i64, _vp],
    "fluidml_hip_squeeze": [_T, _T, _i64p, _i32, _vp],
    "fluidml_hip_unsqueeze": [_T, _T, _i64p, _i32, _vp],
    "fluidml_hip_slice": [_T, _T, _i64p, _i64p, _i64p, _i32, _vp],
    "fluidml_hip_concat2": [_T, _T, _T, _i64, _vp],
    "fluidml_hip_pad": [_T, _T, _i64p, _i32, _u32, _vp],
    "fluidml_hip_pad_view_copy": [_T, _i64p, _i64p, _i32, _i64, _i64p, _T, _vp],
    "fluidml_hip_gather_constant_index_scalar": [_T, _T, _i64, _i64, _u32, _vp],
    "fluidml_hip_gather_constant_indices_tensor": [_T, _T, _T, _i64, _vp],
    "fluidml_hip_gather_constant_data_tensor": [_T, _T, _T, _vp],
    "fluidml_hip_gather_constant_data_tensor_add": [_T, _T, _T, _T, _vp],
    "fluidml_hip_gather_constant_data_tensor_add_tensor_lhs_add_tensor_lhs": [_T, _T, _T, _T, _T, _vp],
    "fluidml_hip_cum_sum": [_T, _T, _i64, _vp],
    # row reductions
    "fluidml_hip_softmax": [_T, _T, _vp, _sz, _i64, _vp],
    "fluidml_hip_layer_normalization_constant_scale_bias": [_T, _T, _T, _T, _vp, _sz, _i64, _f64, _u32, _vp],
    "fluidml_hip_reduce_mean": [_T, _T, _i64p, _i32, _vp],
    "fluidml_hip_max_pool_without_padding": [_T, _T, _i64p, _i64p, _i32, _vp],
    "fluidml_hip_average_pool_without_padding": [_T, _T, _i64p, _i64p, _i32, _vp],
    # contractions
    "fluidml_hip_matmul": [_T, _T, _T, _vp],
    "fluidml_hip_matmul_no_alloc": [_T, _T, _T, _vp],
    "fluidml_hip_matmul_bf16": [_T, _T, _T, _vp],
    "fluidml_hip_gemm_constant_weights_bias": [_T, _T, _T, _T, _f64, _f64, _i32, _i32, _u32, _vp],
    "fluidml_hip_matmul_add": [_T, _T, _T, _T, _vp],
    "fluidml_hip_matmul_chain": [_T, _T, _T, _T, _vp, _u32, _vp],
    "fluidml_hip_matmul_chain_add": [_T, _T, _T, _T, _vp, _T, _T, _u32, _vp],
    "fluidml_hip_matmul_chain_view": [_T, _T, _T, _T, _i64, _i64, _vp, _u32, _vp],
    "fluidml_hip_matmul_chain_group": [_i32, _T, _vp, _vp, _vp, _i64, _i64p, _vp, _u32, _vp],
    "fluidml_hip_matmul_chain_group_norm": [_i32, _T, _vp, _vp, _vp, _vp, _i64, _i64p, _vp, _T, _vp, _u32, _vp],
    "fluidml_hip_gemm_chain": [_T, _T, _T, _T, _f64, _f64, _i32, _i32, _vp, _u32, _vp],
    "fluidml_hip_conv_chain": [_T, _T, _T, _T, _i64p, _i64p, _i64p, _i64, _vp, _u32, _vp],
    "fluidml_hip_conv_chain_scale_add": [_T, _T, _T, _T, _i64p, _i64p, _i64p, _i64, _vp, _T, _T, _u32, _vp],
    "fluidml_hip_conv_chain_mean": [_T, _T, _T, _T, _i64p, _i64p, _i64p, _i64, _vp, _T, _u32, _vp],
    "fluidml_hip_pointwise_conv_pair": [_T, _T, _T, _vp, _T, _T, _vp, _T, _vp],
    "fluidml_hip_softmax_matvec": [_T, _T, _T, _vp],
    "fluidml_hip_elementwise_chain": [_T, _T, _vp, _vp],
    "fluidml_hip_attention": [_T, _T, _T, _T, _f64, _i32, _T, _T, _f64, _vp],
    "fluidml_hip_div_add_softmax": [_T, _f64, _T, _T, _i64, _vp],
    "fluidml_hip_add_layer_normalization": [_T, _T, _T, _T, _T, _i64, _f64, _vp],
    "fluidml_hip_gather_constant_data_tensor_stats": [_T, _T, _T, _vp, _vp],
    "fluidml_hip_gather_add_layer_normalization": [_T, _T, _T, _T, _T, _T, _T, _T, _f64, _vp],
    "fluidml_hip_conv_without_padding": [_T, _T, _T, _T, _i64p, _i64p, _i64, _u32, _vp],
    "fluidml_hip_conv_with_padding": [_T, _T, _T, _T, _vp, _sz, _i64p, _i64p, _i64p, _i64, _u32, _vp],
}

for _name, _argtypes in SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError here = the library does not export a declared symbol
    _fn.argtypes = _argtypes
    _fn.restype = ctypes.c_int
lib.fluidml_hip_error_string.argtypes = [ctypes.c_int]
lib.fluidml_hip_error_string.restype = ctypes.c_char_p


(EW_ADD_C, EW_RSUB_C, EW_MUL_C, EW_DIV_C, EW_POW_C, EW_ERF, EW_RELU, EW_TANH, EW_SQRT, EW_NEG, EW_ADD_X, EW_MUL_X,
 EW_SUB_X, EW_RSUB_X, EW_DIV_X, EW_RDIV_X) = range(16)


class FlEwProgram(ctypes.Structure):
    """fl_ew_program of include/fluidml_hip.h"""
    _fields_ = [("n", ctypes.c_int32), ("op", ctypes.c_int32 * 8), ("c", ctypes.c_float * 8)]


class FlNormFusion(ctypes.Structure):
    """fl_norm_fusion of include/fluidml_hip.h"""
    _fields_ = [("deferred", ctypes.c_int32), ("width", ctypes.c_int32), ("epsilon", ctypes.c_double),
                ("stats", ctypes.c_void_p), ("scale", ctypes.POINTER(FlTensor)), ("shift", ctypes.POINTER(FlTensor)),
                ("stats_out", ctypes.c_void_p), ("addend2", ctypes.POINTER(FlTensor))]


FL_NORM_NONE, FL_NORM_LHS, FL_NORM_ADDEND = 0, 1, 2


def make_chain(steps) -> FlEwProgram:
    """steps: sequence of (op, constant) pairs"""
    g = FlEwProgram()
    g.n = len(steps)
    for i, (op, c) in enumerate(steps):
        g.op[i] = op
        g.c[i] = c
    return g


def error_string(code: int) -> str:
    return lib.fluidml_hip_error_string(int(code)).decode()


def check(code: int, what: str = "fluidml_hip call") -> None:
    if code != 0:
        raise FluidmlHipError(code, what)


def call(name: str, *args) -> None:
    """Call entry point ``fluidml_hip_<name>`` and raise on a non-zero return code."""
    full = name if name.startswith("fluidml_hip_") else "fluidml_hip_" + name
    check(getattr(lib, full)(*args), full)


def default_layout(rank: int) -> list:
    return list(range(rank))


def physical_shape(shape: Sequence[int], layout: Sequence[int]) -> list:
    """physical_shape[layout[i]] = shape[i] (reference utils.cpp:64-76)."""
    phys = [0] * len(shape)
    for i, j in enumerate(layout):
        phys[j] = int(shape[i])
    return phys


def row_major_strides(shape: Sequence[int]) -> list:
    strides = [1] * len(shape)
    for i in range(len(shape) - 1, 0, -1):
        strides[i - 1] = strides[i] * int(shape[i])
    return strides


def layout_strides(shape: Sequence[int], layout: Optional[Sequence[int]] = None) -> list:
    """Element strides of a tensor stored with `layout` (reference utils.cpp:85-102)."""
    if layout is None:
        layout = default_layout(len(shape))
    phys = row_major_strides(physical_shape(shape, layout))
    return [phys[j] for j in layout]


def make_tensor(base: int, dtype: int, shape: Sequence[int], strides: Optional[Sequence[int]] = None) -> FlTensor:
    if len(shape) > FL_MAX_RANK:
        raise ValueError(f"rank {len(shape)} exceeds FL_MAX_RANK={FL_MAX_RANK}")
    if strides is None:
        strides = row_major_strides(shape)
    t = FlTensor()
    t.base = int(base)
    t.dtype = int(dtype)
    t.rank = len(shape)
    for i, (s, st) in enumerate(zip(shape, strides)):
        t.shape[i] = int(s)
        t.strides[i] = int(st)
    return t


def i64_array(values: Iterable[int]):
    vals = [int(v) for v in values]
    return (ctypes.c_int64 * max(len(vals), 1))(*vals)

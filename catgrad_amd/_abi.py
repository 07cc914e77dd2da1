"""ctypes view of the C ABI declared in include/catgrad_hip.h.

The same binding serves any shared library that exports the ABI; the package
itself only ever loads the HIP library (see `catgrad_amd.backend`).
"""
from __future__ import annotations

import ctypes as C

MAX_RANK = 8

# enum cg_dtype — order of `enum Dtype` (catgrad/src/category/core.rs:23-29)
F32, F16, BF16, F8, U32 = 0, 1, 2, 3, 4
DTYPE_NAMES = {F32: "f32", F16: "f16", BF16: "bf16", F8: "f8", U32: "u32"}

# enum cg_status
OK, ERR_SHAPE, ERR_DTYPE, ERR_RANGE, ERR_DEVICE, ERR_UNSUPPORTED, ERR_ARG = range(7)

# enum cg_unary_op / cg_binary_op
NEG, SIN, COS, EXP, LOG, FLOOR, ROUND = range(7)
ADD, SUB, MUL, DIV, POW, LT, GT, GTE, LTE, EQ = range(10)

# enum cg_kernel_class
K_GEMM_MFMA, K_GEMM_SKINNY, K_GEMM_SIMPLE, K_ELEMENTWISE, K_REDUCE, K_GATHER, K_ATTENTION, K_PACK = range(8)

_P = C.c_void_p
_PP = C.POINTER(C.c_void_p)
_SZ = C.c_size_t
_SZP = C.POINTER(C.c_size_t)
_I = C.c_int

# name -> (restype, argtypes); every symbol the header declares.
SIGNATURES = {
    "cg_backend_create": (_I, [_I, _PP]),
    "cg_backend_destroy": (None, [_P]),
    "cg_last_error": (C.c_char_p, []),
    "cg_backend_name": (C.c_char_p, [_P]),
    "cg_sync": (_I, [_P]),
    "cg_pool_stats": (_I, [_P, _SZP, _SZP]),
    "cg_pool_trim": (_I, [_P]),
    "cg_profile_enable": (_I, [_P, _I, C.c_uint]),
    "cg_realize": (_I, [_P, _P]),
    "cg_program_stats": (_I, [_P, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64), _I]),
    "cg_profile_read": (_I, [_P, _I, C.POINTER(C.c_uint64), C.POINTER(C.c_double), C.POINTER(C.c_double), _I]),
    "cg_tensor_retain": (None, [_P]),
    "cg_tensor_release": (None, [_P]),
    "cg_tensor_rank": (_SZ, [_P]),
    "cg_tensor_shape": (None, [_P, _SZP]),
    "cg_tensor_dtype": (_I, [_P]),
    "cg_tensor_numel": (_SZ, [_P]),
    "cg_tensor_is_contiguous": (_I, [_P]),
    "cg_zeros": (_I, [_P, _I, _SZP, _SZ, _PP]),
    "cg_from_host": (_I, [_P, _I, _P, _SZ, _SZP, _SZ, _PP]),
    "cg_from_host_bf16_as_f32": (_I, [_P, _P, _SZ, _SZP, _SZ, _PP]),
    "cg_arange": (_I, [_P, _SZ, _PP]),
    "cg_to_host": (_I, [_P, _P, _P, _SZ]),
    "cg_to_bool": (_I, [_P, _P, C.POINTER(_I)]),
    "cg_compare": (_I, [_P, _P, _P, C.POINTER(_I)]),
    "cg_format_tensor": (_I, [_P, _P, C.c_char_p, _SZ]),
    "cg_cast": (_I, [_P, _P, _I, _PP]),
    "cg_unary": (_I, [_P, _I, _P, _PP]),
    "cg_binary": (_I, [_P, _I, _P, _P, _PP]),
    "cg_where": (_I, [_P, _P, _P, _P, _PP]),
    "cg_matmul": (_I, [_P, _P, _P, _PP]),
    "cg_sum": (_I, [_P, _P, _PP]),
    "cg_max": (_I, [_P, _P, _PP]),
    "cg_argmax": (_I, [_P, _P, _PP]),
    "cg_noalloc_setup": (_I, [_I]),
    "cg_argmax_rows_noalloc": (_I, [_I, _I, _P, _SZ, _SZ, _P, _P]),
    "cg_topk": (_I, [_P, _P, _SZ, _PP, _PP]),
    "cg_broadcast": (_I, [_P, _P, _SZP, _SZ, _PP]),
    "cg_reshape": (_I, [_P, _P, _SZP, _SZ, _PP]),
    "cg_transpose": (_I, [_P, _P, _SZ, _SZ, _PP]),
    "cg_slice": (_I, [_P, _P, _SZ, _SZ, _SZ, _PP]),
    "cg_concat": (_I, [_P, _P, _P, _SZ, _PP]),
    "cg_index": (_I, [_P, _P, _SZ, _P, _PP]),
}


def bind(path: str) -> C.CDLL:
    """dlopen `path` (RTLD_LOCAL) and attach the ABI's signatures.

    Raises AttributeError naming the first missing symbol."""
    lib = C.CDLL(path, mode=C.RTLD_LOCAL)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


def dims_array(shape):
    shape = tuple(int(s) for s in shape)
    arr = (C.c_size_t * max(len(shape), 1))(*shape)
    return arr, len(shape)

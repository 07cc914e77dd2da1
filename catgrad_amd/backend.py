"""Python mirror of catgrad's interpreter `Backend` trait over the C ABI.

Method names, argument order and failure behaviour follow
`catgrad/src/interpreter/backend/mod.rs:24-122`; where the trait takes a
`TaggedTensorTuple<Self, N>` the Python method takes N tensors.  The Rust trait
moves its arguments; here an argument is borrowed unless it is wrapped with
`Tensor.move()`, in which case the Python object gives up its reference (the
library then sees a uniquely owned operand exactly as the Rust caller would).

`HipBackend` is the product: it loads `libcatgrad_hip.so` built from
`catgrad_amd/csrc` and raises if that library is missing or no GPU is usable.
There is no CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

from . import _abi as A

_HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIBRARY = os.path.join(_HERE, "csrc", "libcatgrad_hip.so")


class BackendPanic(RuntimeError):
    """A failure the reference reports by panicking (shape mismatch, bad axis, ...)."""

    def __init__(self, status: int, message: str):
        super().__init__(message)
        self.status = status


class ShapeError(BackendPanic):
    """`BackendError::ShapeError` (backend/mod.rs:129-132): data length != shape size."""


class _Moved:
    __slots__ = ("handle",)

    def __init__(self, handle):
        self.handle = handle


class Tensor:
    """`Backend::BackendTensor`: a reference-counted handle.  `clone()` is O(1)."""

    __slots__ = ("_be", "_h")

    def __init__(self, be: "Backend", handle: int):
        self._be = be
        self._h = handle

    # BackendTensorOps::shape (backend/mod.rs:124-126)
    @property
    def shape(self) -> tuple:
        if self._h is None:
            raise ValueError("use of a moved tensor")
        lib = self._be._lib
        r = lib.cg_tensor_rank(self._h)
        buf = (C.c_size_t * max(r, 1))()
        lib.cg_tensor_shape(self._h, buf)
        return tuple(int(buf[i]) for i in range(r))

    @property
    def dtype(self) -> int:
        if self._h is None:
            raise ValueError("use of a moved tensor")
        return int(self._be._lib.cg_tensor_dtype(self._h))

    @property
    def is_contiguous(self) -> bool:
        if self._h is None:
            raise ValueError("use of a moved tensor")
        return bool(self._be._lib.cg_tensor_is_contiguous(self._h))

    def clone(self) -> "Tensor":
        if self._h is None:
            raise ValueError("use of a moved tensor")
        self._be._lib.cg_tensor_retain(self._h)
        return Tensor(self._be, self._h)

    def move(self) -> _Moved:
        """Give this object's reference to the next op (Rust's pass-by-value)."""
        h, self._h = self._h, None
        if h is None:
            raise ValueError("tensor was already moved")
        return _Moved(h)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h is not None and self._be is not None and self._be._lib is not None:
            self._be._lib.cg_tensor_release(h)

    def __repr__(self):
        if self._h is None:
            return "Tensor(<moved>)"
        return f"Tensor({A.DTYPE_NAMES[self.dtype]}{list(self.shape)})"


class Backend:
    """Trait `Backend` over a bound ABI library (`_abi.bind`)."""

    def __init__(self, lib, device: int = 0):
        self._lib = lib
        out = C.c_void_p()
        st = lib.cg_backend_create(device, C.byref(out))
        if st != A.OK:
            raise BackendPanic(st, lib.cg_last_error().decode())
        self._b = out.value

    def close(self):
        if self._lib is not None and self._b is not None:
            self._lib.cg_backend_destroy(self._b)
            self._b = None

    @property
    def name(self) -> str:
        return self._lib.cg_backend_name(self._b).decode()

    # ---- plumbing -----------------------------------------------------------
    def _check(self, st: int):
        if st != A.OK:
            msg = self._lib.cg_last_error().decode()
            raise (ShapeError if msg == "ShapeError" else BackendPanic)(st, msg)

    def _take(self, t) -> int:
        if isinstance(t, _Moved):
            return t.handle
        if t._h is None:
            raise ValueError("use of a moved tensor")
        self._lib.cg_tensor_retain(t._h)
        return t._h

    def _op(self, fn, *args) -> Tensor:
        out = C.c_void_p()
        self._check(fn(self._b, *args, C.byref(out)))
        return Tensor(self, out.value)

    def sync(self):
        self._check(self._lib.cg_sync(self._b))

    def pool_stats(self):
        u, c = C.c_size_t(), C.c_size_t()
        self._check(self._lib.cg_pool_stats(self._b, C.byref(u), C.byref(c)))
        return int(u.value), int(c.value)

    def realize(self, x: "Tensor") -> "Tensor":
        """Queue the computation of a lazily evaluated element-wise result now."""
        self._check(self._lib.cg_realize(self._b, x._h))
        return x

    def program_stats(self, reset: bool = True):
        """(compiled, interpreted) launches of fused programs since the last reset."""
        c, i = C.c_uint64(), C.c_uint64()
        self._check(self._lib.cg_program_stats(self._b, C.byref(c), C.byref(i), int(reset)))
        return int(c.value), int(i.value)

    def profile_enable(self, cls: int, sample_every: int = 1):
        """Time every `sample_every`-th launch of a kernel class with HIP events (0: off)."""
        self._check(self._lib.cg_profile_enable(self._b, cls, sample_every))

    def profile_read(self, cls: int, reset: bool = True):
        """(launches timed, device milliseconds, algorithmic work) of a kernel class."""
        n, ms, w = C.c_uint64(), C.c_double(), C.c_double()
        self._check(self._lib.cg_profile_read(self._b, cls, C.byref(n), C.byref(ms), C.byref(w), int(reset)))
        return int(n.value), float(ms.value), float(w.value)

    def pool_trim(self):
        self._check(self._lib.cg_pool_trim(self._b))

    # ---- creation -------------------------------------------------------------
    def zeros(self, shape, target_dtype: int) -> Tensor:
        d, r = A.dims_array(shape)
        return self._op(lambda b, o: self._lib.cg_zeros(b, target_dtype, d, r, o))

    def _from_vec(self, dtype, npdtype, data, shape) -> Tensor:
        arr = np.ascontiguousarray(np.asarray(data, dtype=npdtype).reshape(-1))
        d, r = A.dims_array(shape)
        ptr = arr.ctypes.data_as(C.c_void_p)
        return self._op(lambda b, o: self._lib.cg_from_host(b, dtype, ptr, arr.size, d, r, o))

    def ndarray_from_vec_f32(self, data, shape) -> Tensor:
        return self._from_vec(A.F32, np.float32, data, shape)

    def ndarray_from_vec_u32(self, data, shape) -> Tensor:
        return self._from_vec(A.U32, np.uint32, data, shape)

    def ndarray_from_vec_f16(self, data, shape) -> Tensor:
        return self._from_vec(A.F16, np.float16, data, shape)

    def ndarray_from_vec_bf16(self, data, shape) -> Tensor:
        return self._from_vec(A.BF16, np.uint16, data, shape)

    def ndarray_from_vec_fp8(self, data, shape) -> Tensor:
        return self._from_vec(A.F8, np.uint8, data, shape)

    def from_bf16_bits(self, bits, shape) -> Tensor:
        """Weight ingest (catgrad-llm/src/utils/mod.rs:158-168): an f32 tensor from bfloat16 bit
        patterns (uint16); the widening happens in the backend."""
        arr = np.ascontiguousarray(np.asarray(bits, dtype=np.uint16).reshape(-1))
        d, r = A.dims_array(shape)
        ptr = arr.ctypes.data_as(C.c_void_p)
        return self._op(lambda b, o: self._lib.cg_from_host_bf16_as_f32(b, ptr, arr.size, d, r, o))

    def from_numpy(self, arr) -> Tensor:
        """`interpreter::tensor` (catgrad/src/interpreter/mod.rs:23-33) for a numpy array."""
        arr = np.asarray(arr)
        if arr.dtype == np.float32:
            return self.ndarray_from_vec_f32(arr, arr.shape)
        if arr.dtype == np.uint32:
            return self.ndarray_from_vec_u32(arr, arr.shape)
        if arr.dtype == np.float16:
            return self.ndarray_from_vec_f16(arr, arr.shape)
        raise TypeError(f"unsupported dtype {arr.dtype} (bfloat16: ndarray_from_vec_bf16 with uint16 bit patterns)")

    def arange(self, end: int) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_arange(b, end, o))

    # ---- read-back --------------------------------------------------------------
    def to_vec(self, x: Tensor) -> np.ndarray:
        """`Backend::to_vec`: flat row-major contents."""
        n = int(self._lib.cg_tensor_numel(x._h))
        # f16 as numpy float16; bf16 as its uint16 bit patterns (numpy has no bfloat16): `bits << 16` is the f32 value;
        # fp8 (E4M3) as its uint8 bit patterns
        out = np.empty(n, dtype={A.F32: np.float32, A.F16: np.float16, A.BF16: np.uint16, A.F8: np.uint8}.get(x.dtype, np.uint32))
        self._check(self._lib.cg_to_host(self._b, x._h, out.ctypes.data_as(C.c_void_p), n))
        return out

    def to_numpy(self, x: Tensor) -> np.ndarray:
        """Logical contents with shape.  Goes through `reshape` to the same shape first,
        which yields a contiguous tensor on every backend (NdArrayBackend's `to_vec`
        refuses non-contiguous views, ndarray.rs:52)."""
        shp = x.shape
        y = x if x.is_contiguous else self.reshape(x, shp)
        return self.to_vec(y).reshape(shp)

    def to_bool(self, x: Tensor) -> bool:
        out = C.c_int()
        self._check(self._lib.cg_to_bool(self._b, x._h, C.byref(out)))
        return bool(out.value)

    def compare(self, x: Tensor, y: Tensor) -> bool:
        out = C.c_int()
        self._check(self._lib.cg_compare(self._b, x._h, y._h, C.byref(out)))
        return bool(out.value)

    def format_tensor(self, x: Tensor) -> str:
        buf = C.create_string_buffer(4096)
        self._check(self._lib.cg_format_tensor(self._b, x._h, buf, len(buf)))
        return buf.value.decode()

    # ---- element-wise -------------------------------------------------------------
    def cast(self, x, target_dtype: int) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_cast(b, self._take(x), target_dtype, o))

    def _unary(self, op, x) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_unary(b, op, self._take(x), o))

    def _binary(self, op, x, y) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_binary(b, op, self._take(x), self._take(y), o))

    def neg(self, x): return self._unary(A.NEG, x)
    def sin(self, x): return self._unary(A.SIN, x)
    def cos(self, x): return self._unary(A.COS, x)
    def exp(self, x): return self._unary(A.EXP, x)
    def log(self, x): return self._unary(A.LOG, x)
    def floor(self, x): return self._unary(A.FLOOR, x)
    def round(self, x): return self._unary(A.ROUND, x)

    def add(self, x, y): return self._binary(A.ADD, x, y)
    def sub(self, x, y): return self._binary(A.SUB, x, y)
    def mul(self, x, y): return self._binary(A.MUL, x, y)
    def div(self, x, y): return self._binary(A.DIV, x, y)
    def pow(self, x, y): return self._binary(A.POW, x, y)
    def lt(self, x, y): return self._binary(A.LT, x, y)
    def gt(self, x, y): return self._binary(A.GT, x, y)
    def gte(self, x, y): return self._binary(A.GTE, x, y)
    def lte(self, x, y): return self._binary(A.LTE, x, y)
    def eq(self, x, y): return self._binary(A.EQ, x, y)

    def where_cond(self, mask, x, y) -> Tensor:
        return self._op(
            lambda b, o: self._lib.cg_where(b, self._take(mask), self._take(x), self._take(y), o)
        )

    # ---- contraction / reductions ----------------------------------------------------
    def matmul(self, x, y) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_matmul(b, self._take(x), self._take(y), o))

    def sum(self, x): return self._op(lambda b, o: self._lib.cg_sum(b, self._take(x), o))
    def max(self, x): return self._op(lambda b, o: self._lib.cg_max(b, self._take(x), o))
    def argmax(self, x): return self._op(lambda b, o: self._lib.cg_argmax(b, self._take(x), o))

    def topk(self, x, k: int):
        v, i = C.c_void_p(), C.c_void_p()
        self._check(self._lib.cg_topk(self._b, self._take(x), k, C.byref(v), C.byref(i)))
        return Tensor(self, v.value), Tensor(self, i.value)

    # ---- shape / indexing ---------------------------------------------------------------
    def broadcast(self, x, shape) -> Tensor:
        d, r = A.dims_array(shape)
        return self._op(lambda b, o: self._lib.cg_broadcast(b, self._take(x), d, r, o))

    def reshape(self, x, new_shape) -> Tensor:
        d, r = A.dims_array(new_shape)
        return self._op(lambda b, o: self._lib.cg_reshape(b, self._take(x), d, r, o))

    def transpose(self, x, dim0: int, dim1: int) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_transpose(b, self._take(x), dim0, dim1, o))

    def slice(self, x, dim: int, start: int, len: int) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_slice(b, self._take(x), dim, start, len, o))

    def concat(self, x, y, dim: int) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_concat(b, self._take(x), self._take(y), dim, o))

    def index(self, x, dim: int, indices) -> Tensor:
        return self._op(lambda b, o: self._lib.cg_index(b, self._take(x), dim, self._take(indices), o))


_hip_lib = None


def load_hip_library():
    """Bind the in-tree HIP library; loud failure when it has not been built."""
    global _hip_lib
    if _hip_lib is None:
        if not os.path.exists(HIP_LIBRARY):
            raise RuntimeError(
                f"{HIP_LIBRARY} is missing: build it with `make -C {os.path.dirname(HIP_LIBRARY)}` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`). There is no CPU fallback."
            )
        try:  # a process that also uses torch must hold ONE HIP runtime, torch's: torch goes first when it is there
            import torch  # noqa: F401
        except ImportError:
            pass
        _hip_lib = A.bind(HIP_LIBRARY)
    return _hip_lib


class HipBackend(Backend):
    """The MI355X backend: `HipBackend` in place of `NdArrayBackend`."""

    def __init__(self, device: int = 0):
        super().__init__(load_hip_library(), device)

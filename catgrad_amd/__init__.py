"""catgrad_amd — MI355X (gfx950) implementation of catgrad's interpreter `Backend`.

Public surface:
  HipBackend   — the trait implementation (hand-written HIP kernels behind a C ABI)
  Tensor       — its `BackendTensor`
  dtype / op constants re-exported from `_abi`
"""
from ._abi import F32, F16, BF16, F8, U32  # noqa: F401
from .backend import Backend, BackendPanic, HipBackend, ShapeError, Tensor  # noqa: F401

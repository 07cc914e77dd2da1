"""Tensor handles may outlive the backend that made them, as the reference's tensors do (they own their data;
`BackendTensorOps: Send + Sync + Clone`, catgrad/src/interpreter/backend/mod.rs:124-126): releasing — or cloning and
then releasing — the last handle after `cg_backend_destroy` is safe.  Host-side lifetime only: every kernel has
finished by the time the backend is destroyed.  Runs on the oracle library on the CPU and on the HIP library under
`-m gpu`, through the C ABI."""
import ctypes as C

import numpy as np
import pytest

from catgrad_amd import _abi as A


def _survivors(lib):
    b = C.c_void_p()
    assert lib.cg_backend_create(0, C.byref(b)) == A.OK, lib.cg_last_error().decode()

    def from_np(a):
        d, r = A.dims_array(a.shape)
        out = C.c_void_p()
        assert lib.cg_from_host(b, A.F32, a.ctypes.data_as(C.c_void_p), a.size, d, r, C.byref(out)) == A.OK
        return out

    x = from_np(np.arange(4096, dtype=np.float32).reshape(64, 64))
    y = from_np(np.ones((64, 64), np.float32))
    lib.cg_tensor_retain(x)
    lib.cg_tensor_retain(y)
    z = C.c_void_p()   # a deferred result that is never computed: it holds x and y through its program
    assert lib.cg_binary(b, A.ADD, x, y, C.byref(z)) == A.OK
    lib.cg_tensor_retain(x)
    v = C.c_void_p()   # a view sharing x's buffer
    assert lib.cg_transpose(b, x, 0, 1, C.byref(v)) == A.OK
    s = C.c_void_p()   # a constant that never had device memory
    d, r = A.dims_array((3, 5))
    assert lib.cg_zeros(b, A.U32, d, r, C.byref(s)) == A.OK
    host = np.zeros(4096, np.float32)
    assert lib.cg_to_host(b, x, host.ctypes.data_as(C.c_void_p), 4096) == A.OK, lib.cg_last_error().decode()
    np.testing.assert_array_equal(host, np.arange(4096, dtype=np.float32))
    return b, [x, y, z, v, s]


def _destroy_then_release(lib):
    b, handles = _survivors(lib)
    lib.cg_backend_destroy(b)                       # the owner goes first
    assert lib.cg_tensor_rank(handles[3]) == 2      # shape queries need no backend
    dims = (C.c_size_t * 2)()
    lib.cg_tensor_shape(handles[4], dims)
    assert (dims[0], dims[1]) == (3, 5)
    lib.cg_tensor_retain(handles[0])                # Clone after the backend is gone
    lib.cg_tensor_release(handles[0])
    for h in handles:                               # Drop, in creation order; the last one tears the backend down
        lib.cg_tensor_release(h)
    # the library still works afterwards
    b2, hs = _survivors(lib)
    for h in reversed(hs):
        lib.cg_tensor_release(h)
    lib.cg_backend_destroy(b2)                      # and the ordinary order still does


def _calls_after_destroy_fail(lib):
    """While surviving handles keep a destroyed backend's memory alive, calls on it are refused, not undefined."""
    b, handles = _survivors(lib)
    lib.cg_backend_destroy(b)
    host = np.zeros(4096, np.float32)
    assert lib.cg_to_host(b, handles[0], host.ctypes.data_as(C.c_void_p), 4096) == A.ERR_ARG
    assert "cg_backend_destroy" in lib.cg_last_error().decode()
    out = C.c_void_p()
    lib.cg_tensor_retain(handles[0])
    assert lib.cg_unary(b, A.NEG, handles[0], C.byref(out)) == A.ERR_ARG   # (the consumed reference is dropped)
    assert lib.cg_sync(b) == A.ERR_ARG
    for h in handles:
        lib.cg_tensor_release(h)


def test_release_after_destroy_oracle():
    from oracle_loader import oracle_library

    _destroy_then_release(oracle_library())


@pytest.mark.gpu
def test_release_after_destroy_hip():
    from catgrad_amd.backend import load_hip_library

    _destroy_then_release(load_hip_library())


@pytest.mark.gpu
def test_calls_on_a_destroyed_backend_fail_hip():
    from catgrad_amd.backend import load_hip_library

    _calls_after_destroy_fail(load_hip_library())

"""The arg-max entry point for callers that cannot allocate (`cg_argmax_rows_noalloc`), through the C ABI:
its output against `cg_argmax`'s (the existing entry point, which takes its scratch from the pool) and against
the CPU oracle, bit-exact (indices), on calls in a row that share the library's fixed scratch array — the
second smaller than the first — and its size limit.

Device memory for the raw-pointer arguments comes from torch (plumbing only): the entry point itself takes plain
addresses and a stream and allocates nothing."""
import ctypes as C

import numpy as np
import pytest
import torch  # before the HIP library is loaded: both then share the one HIP runtime that torch ships

from catgrad_amd import _abi as A

pytestmark = pytest.mark.gpu


def _inputs(seed, rows, n, dtype):
    r = np.random.default_rng(seed)
    if dtype == A.U32:
        x = r.integers(0, 1000, size=(rows, n), dtype=np.uint64).astype(np.uint32)  # many equal maxima
    else:
        x = r.standard_normal((rows, n)).astype(np.float32)
        x[:, ::7] = np.float32(2.5)             # ties: the last of equal maxima wins
        if n > 40:
            x[0, 5] = np.float32(np.nan)        # +NaN is greatest in total order
            x[rows - 1, n - 3] = np.float32(-0.0)
    return x


def _noalloc(lib, x_dev, rows, n, dtype, out_dev):
    rc = lib.cg_argmax_rows_noalloc(0, dtype, C.c_void_p(x_dev.data_ptr()), rows, n, C.c_void_p(out_dev.data_ptr()),
                                    C.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == A.OK, lib.cg_last_error().decode()


@pytest.mark.parametrize("dtype", [A.F32, A.U32])
def test_no_alloc_argmax_matches_the_allocating_entry_point(hip, oracle, dtype):
    lib = hip._lib
    # two calls in a row on the shared scratch array, the second with a smaller input; then a ragged one
    shapes = [(4, 128256), (2, 5000), (3, 1023), (64, 262144 // 4 + 3), (1, 1)]
    out_dev = torch.zeros(64, dtype=torch.int32, device="cuda:0")
    for i, (rows, n) in enumerate(shapes):
        print(f"no_alloc argmax dtype={dtype} rows={rows} n={n}", flush=True)
        x = _inputs(900 + i, rows, n, dtype)
        x_dev = torch.from_numpy(x.view(np.int32)).to("cuda:0")
        out_dev.fill_(-1)
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated(0)
        _noalloc(lib, x_dev, rows, n, dtype, out_dev)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated(0) == before
        got = out_dev[:rows].cpu().numpy().astype(np.uint32)
        # the existing entry point on the same values, and the CPU oracle
        ref = hip.to_numpy(hip.argmax(hip.from_numpy(x))).reshape(rows)
        chk = oracle.to_numpy(oracle.argmax(oracle.from_numpy(x))).reshape(rows)
        np.testing.assert_array_equal(got, ref)
        np.testing.assert_array_equal(got, chk)
        assert (out_dev[rows:].cpu().numpy() == -1).all()   # nothing written beyond the rows asked for


def test_no_alloc_argmax_rejects_what_does_not_fit(hip):
    lib = hip._lib
    x_dev = torch.zeros(16, dtype=torch.float32, device="cuda:0")
    out_dev = torch.zeros(16, dtype=torch.int32, device="cuda:0")
    # 65 rows of 262144 elements: 65 x 256 segments > 16384 partial results
    rc = lib.cg_argmax_rows_noalloc(0, A.F32, C.c_void_p(x_dev.data_ptr()), 65, 262144, C.c_void_p(out_dev.data_ptr()), None)
    assert rc == A.ERR_UNSUPPORTED and "scratch" in lib.cg_last_error().decode()
    rc = lib.cg_argmax_rows_noalloc(0, A.F32, C.c_void_p(x_dev.data_ptr()), 4, 0, C.c_void_p(out_dev.data_ptr()), None)
    assert rc == A.ERR_SHAPE
    rc = lib.cg_argmax_rows_noalloc(0, 9, C.c_void_p(x_dev.data_ptr()), 4, 4, C.c_void_p(out_dev.data_ptr()), None)
    assert rc == A.ERR_UNSUPPORTED
    assert lib.cg_argmax_rows_noalloc(0, A.F32, None, 0, 4, None, None) == A.OK   # no rows: nothing to do

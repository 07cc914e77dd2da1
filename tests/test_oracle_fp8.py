"""Pins of the oracle's fp8 (E4M3) conversions that do not rest on this repository's own formulas: every decoding
and every rounding below 464 against torch.float8_e4m3fn, arithmetic against torch's (which also computes in f32 and
narrows).  Beyond 464 the oracle saturates to 448 as the float8 crate documents, torch gives NaN: not pinned."""
import numpy as np
import pytest
import torch

from catgrad_amd import _abi as A
from cases_fp8 import f8_decode


def torch_bits(x32):
    return torch.from_numpy(np.ascontiguousarray(x32)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def sweep():
    """f32 patterns below 464 in magnitude: random ones, and every exponent of the fp8 range (and some below it) with
    the tie of each of the 8 mantissa steps, just above and just below it."""
    rng = np.random.default_rng(0)
    rand = (rng.standard_normal(200000) * rng.choice([1e-3, 0.05, 1.0, 30.0, 150.0], size=200000)).astype(np.float32)
    exps = np.arange(127 - 14, 127 + 9, dtype=np.uint32) << 23
    steps = (np.arange(8, dtype=np.uint32) << 20)
    tails = np.array([0x00000, 0x00001, 0x7FFFF, 0x80000, 0x80001, 0xFFFFF], dtype=np.uint32)
    grid = (exps[:, None, None] | steps[None, :, None] | tails[None, None, :]).reshape(-1).view(np.float32)
    x = np.concatenate([rand, grid, -grid, np.array([0.0, -0.0, 448.0, 463.99997, -463.99997], np.float32)])
    return x[np.abs(x) < 464.0]


def test_every_pattern_decodes_as_torch(oracle):
    bits = np.arange(256, dtype=np.uint8)
    got = oracle.to_numpy(oracle.cast(oracle.ndarray_from_vec_fp8(bits, bits.shape), A.F32))
    exp = f8_decode(bits)
    assert np.array_equal(np.isnan(got), np.isnan(exp)) and np.isnan(exp).sum() == 2
    np.testing.assert_array_equal(got[~np.isnan(exp)].view(np.uint32), exp[~np.isnan(exp)].view(np.uint32))


def test_rounding_below_464_matches_torch(oracle):
    x = sweep()
    got = oracle.to_numpy(oracle.cast(oracle.from_numpy(x), A.F8))
    np.testing.assert_array_equal(got, torch_bits(x))


def test_saturation_and_nan(oracle):
    x = np.array([464.0, 480.0, 1e9, np.inf, -464.0, -np.inf, np.nan], np.float32)
    got = oracle.to_numpy(oracle.cast(oracle.from_numpy(x), A.F8))
    np.testing.assert_array_equal(got[:6], np.array([0x7E, 0x7E, 0x7E, 0x7E, 0xFE, 0xFE], np.uint8))
    assert got[6] & 0x7F == 0x7F


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_arithmetic_matches_torch(oracle, op):
    rng = np.random.default_rng(3)
    a = rng.integers(0, 256, size=60000).astype(np.uint8)
    b = rng.integers(0, 256, size=60000).astype(np.uint8)
    keep = ((a & 0x7F) != 0x7F) & ((b & 0x7F) != 0x7F) & ((b & 0x7F) != 0)
    a, b = a[keep], b[keep]
    got = oracle.to_numpy(getattr(oracle, op)(oracle.ndarray_from_vec_fp8(a, a.shape), oracle.ndarray_from_vec_fp8(b, b.shape)))
    xa, xb = (torch.from_numpy(v).view(torch.float8_e4m3fn).float() for v in (a, b))
    exact = {"add": xa + xb, "sub": xa - xb, "mul": xa * xb, "div": xa / xb}[op]
    inside = (exact.abs() < 464.0).numpy()
    exp = exact.to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    np.testing.assert_array_equal(got[inside], exp[inside])
    assert np.all((got[~inside] & 0x7F) == 0x7E)

"""Pins of the oracle's 16-bit float dtypes that do not rest on this repository's own formulas.

The oracle writes binary16 and bfloat16 rounding out on bit patterns; here they are checked against two
independent implementations: numpy's float16 (every f32 exponent, ties, subnormals, overflow) and
torch.bfloat16 (conversion and the element-wise arithmetic, which torch's CPU kernels also compute in f32 and
round).  The closed forms used by tests/cases_half.py are checked against torch the same way."""
import numpy as np
import pytest
import torch

from catgrad_amd import BackendPanic
from catgrad_amd import _abi as A
from cases_half import bf16_round_bits, bf16_widen


def torch_bf16_bits(x32):
    return torch.from_numpy(np.ascontiguousarray(x32)).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def sweep():
    """f32 bit patterns: random ones, every exponent with ties / just above / just below them, specials."""
    rng = np.random.default_rng(0)
    rand = rng.integers(0, 2**32, size=200000, dtype=np.uint64).astype(np.uint32)
    exps = np.arange(256, dtype=np.uint32) << 23
    tails = np.array([0x0000, 0x0FFF, 0x1000, 0x1001, 0x2FFF, 0x3000, 0x3001, 0x7FFF, 0x8000, 0x8001, 0x17FFF, 0x18000, 0x18001,
                      0x7FFFFF, 0x7FEFFF, 0x7FF000, 0x7FF001, 0x7F7FFF, 0x7F8000, 0x7F8001], dtype=np.uint32)
    grid = (exps[:, None] | tails[None, :]).reshape(-1)
    allb = np.concatenate([rand, grid, grid | np.uint32(0x80000000)])
    return allb.view(np.float32)


def test_f32_to_f16_matches_numpy(oracle):
    x = sweep()
    got = oracle.to_numpy(oracle.cast(oracle.from_numpy(x), A.F16))
    with np.errstate(over="ignore"):
        exp = x.astype(np.float16)
    nan = np.isnan(exp)
    assert np.array_equal(np.isnan(got), nan)
    np.testing.assert_array_equal(got.view(np.uint16)[~nan], exp.view(np.uint16)[~nan])


def test_f32_to_bf16_matches_torch_and_closed_form(oracle):
    x = sweep()
    got = oracle.to_numpy(oracle.cast(oracle.from_numpy(x), A.BF16))
    exp = torch_bf16_bits(x)
    nan = np.isnan(x)
    np.testing.assert_array_equal(got[~nan], exp[~nan])
    assert np.all(np.isnan(bf16_widen(got[nan])))
    np.testing.assert_array_equal(bf16_round_bits(x)[~nan], exp[~nan])


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_bf16_arithmetic_matches_torch(oracle, op):
    rng = np.random.default_rng(3)
    a = bf16_round_bits((rng.standard_normal(50000) * 10).astype(np.float32))
    b = bf16_round_bits((rng.standard_normal(50000) * 10).astype(np.float32))
    ta, tb = (oracle.ndarray_from_vec_bf16(v, v.shape) for v in (a, b))
    got = oracle.to_numpy(getattr(oracle, op)(ta, tb))
    xa, xb = (torch.from_numpy(v.view(np.int16)).view(torch.bfloat16) for v in (a, b))
    exp = {"add": xa + xb, "sub": xa - xb, "mul": xa * xb, "div": xa / xb}[op].view(torch.int16).numpy().view(np.uint16)
    np.testing.assert_array_equal(got, exp)


@pytest.mark.parametrize("op", ["add", "sub", "mul", "div"])
def test_f16_arithmetic_matches_numpy(oracle, op):
    rng = np.random.default_rng(4)
    a = (rng.standard_normal(50000) * 30).astype(np.float16)
    b = (rng.standard_normal(50000) * 30).astype(np.float16)
    got = oracle.to_numpy(getattr(oracle, op)(oracle.from_numpy(a), oracle.from_numpy(b)))
    with np.errstate(all="ignore"):
        exp = {"add": a + b, "sub": a - b, "mul": a * b, "div": a / b}[op]
    np.testing.assert_array_equal(got.view(np.uint16), exp.view(np.uint16))


def test_dtype_rules(oracle):
    x = oracle.from_numpy(np.ones((2, 3), np.float32))
    h, bh = oracle.cast(x, A.F16), oracle.cast(x, A.BF16)
    assert (h.dtype, bh.dtype) == (A.F16, A.BF16)
    assert oracle.cast(h, A.F16).dtype == A.F16
    for bad in (lambda: oracle.add(h, bh), lambda: oracle.mul(h, x), lambda: oracle.matmul(h, oracle.transpose(x, 0, 1)),
                lambda: oracle.zeros((2,), 9), lambda: oracle.cast(x, 9), lambda: oracle.add(h, oracle.cast(x, A.F8)),
                lambda: oracle.sin(oracle.cast(h, A.U32))):
        with pytest.raises(BackendPanic):
            bad()
    assert "f16[2,3]" in oracle.format_tensor(h) and "bf16[2,3]" in oracle.format_tensor(bh)

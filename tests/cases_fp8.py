"""Cases for fp8 (`Dtype::F8` = float8::F8E4M3: 1 sign, 4 exponent bits with bias 7, 3 mantissa bits, no infinities,
0x7F / 0xFF are NaN, largest finite 448, subnormals m * 2^-9), appended to `cases.CASES`.

NdArrayBackend has `todo!()` for this dtype (ndarray.rs:7-9); the semantics are those CandleBackend gets from the
float8 crate (candle.rs:9, 382, 553-562, 605-718): widen exactly, compute in f32, narrow with round to nearest even,
saturating at 448 (the crate documents CUDA's `__NV_SATFINITE` conversion).  The closed form below is
torch.float8_e4m3fn for everything that rounds below 464 — torch and the crate agree there — and +-448 beyond, where
torch would give NaN (that part rests on the crate's documentation only: parity unpinned).
Tensors cross the test API as uint8 bit patterns; results are compared as decoded float32 values."""
import numpy as np
import torch

from catgrad_amd import _abi as A
from cases import CASES, Case, argmax_last, f32, u32


def case(name, kind="exact", scale=None):
    def deco(pair):
        run, expect = pair()
        CASES.append(Case(name, run, expect, kind, scale))
        return pair

    return deco


F8_LUT = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()     # decoding of every pattern


def f8_decode(bits):
    return F8_LUT[np.asarray(bits, dtype=np.uint8)]


def f8_round(x):
    """float array -> nearest E4M3 value as float32 (ties to even), +-448 from 464 on, NaN stays NaN."""
    x32 = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    sat = np.abs(x32) >= 464.0
    safe = np.where(sat, np.float32(0), x32)
    r = torch.from_numpy(safe).to(torch.float8_e4m3fn).float().numpy()
    return np.where(sat, np.copysign(np.float32(448), x32), r).astype(np.float32)


def f8_encode(x):
    """Representable float32 values -> uint8 patterns."""
    return torch.from_numpy(np.ascontiguousarray(np.asarray(x, dtype=np.float32))).to(torch.float8_e4m3fn).view(torch.uint8).numpy()


def f8_inputs(seed, shape, scale=1.0):
    """(bit patterns to upload, their float32 values) of random representable numbers."""
    v = f8_round(f32(seed, shape, scale))
    return f8_encode(v), v


def read(be, t):
    """Decoded values of an fp8 tensor (which NaN pattern comes back is not part of the value)."""
    a = be.to_numpy(t)
    assert a.dtype == np.uint8
    return f8_decode(a)


EDGE = np.array([0.0, -0.0, 1.0, -1.0, 448.0, 447.9, 432.0, 440.0, 456.0, 463.9, 464.0, 480.0, -464.0, 1e6, -1e6, 3.4e38, np.inf, -np.inf,
                 np.nan, 2.0 ** -9, 2.0 ** -10, 2.0 ** -10 * 1.0001, 3 * 2.0 ** -10, 2.0 ** -6, 2.0 ** -6 - 2.0 ** -10, 7.5 * 2.0 ** -9,
                 1.0625, 1.1875, 1.0624, 1.0626, 1.3125, 0.3333, 17.0, 19.0, 1e-10, -1e-45], dtype=np.float32)


@case("fp8_all_bit_patterns_roundtrip")
def _():
    bits = np.arange(256, dtype=np.uint8).reshape(16, 16)

    def run(be):
        t = be.ndarray_from_vec_fp8(bits, bits.shape)
        back = be.to_numpy(t)
        nan = (back & 0x7F) == 0x7F
        return [np.where(nan, 0x7F, back).astype(np.uint32), be.to_numpy(be.cast(t, A.F32))]

    def expect():
        nan = (bits & 0x7F) == 0x7F
        return [np.where(nan, 0x7F, bits).astype(np.uint32), f8_decode(bits)]

    return run, expect


@case("fp8_cast_matrix")
def _():
    """f32 -> fp8 rounds to nearest even and saturates; fp8 -> u32 is Rust `as` on the value; u32 -> fp8 goes through
    f32; the 16-bit dtypes hold every fp8 value, and round into it like f32 does."""
    x = np.concatenate([EDGE, f32(900, (4000,), 50.0), f32(901, (4000,), 0.01), f32(902, (2000,), 300.0)])
    n = u32(903, (1000,)) % 600
    bits, vals = f8_inputs(904, (2000,), 100.0)
    h = f32(905, (3000,), 40.0).astype(np.float16)

    def run(be):
        t8 = be.ndarray_from_vec_fp8(bits, bits.shape)
        return [read(be, be.cast(be.from_numpy(x), A.F8)), be.to_numpy(be.cast(t8, A.U32)), read(be, be.cast(be.from_numpy(n), A.F8)),
                be.to_numpy(be.cast(t8, A.F16)).astype(np.float32), read(be, be.cast(be.from_numpy(h), A.F8)),
                be.to_numpy(be.cast(be.cast(t8, A.BF16), A.F32)), be.to_numpy(be.cast(t8, A.F32))]

    def expect():
        return [f8_round(x), np.where(vals > 0, np.floor(vals), 0).astype(np.uint32), f8_round(n.astype(np.float32)), vals,
                f8_round(h.astype(np.float32)), vals, vals]

    return run, expect


@case("fp8_arithmetic")
def _():
    ab, av = f8_inputs(910, (64, 130), 12.0)
    bb, bv = f8_inputs(911, (64, 130), 12.0)
    bv = np.where(bv == 0, np.float32(0.5), bv)
    bb = f8_encode(bv)

    def run(be):
        a, b = be.ndarray_from_vec_fp8(ab, ab.shape), be.ndarray_from_vec_fp8(bb, bb.shape)
        outs = [read(be, getattr(be, op)(a, b)) for op in ("add", "sub", "mul", "div")]
        outs += [read(be, getattr(be, op)(a, b)) for op in ("lt", "gte", "eq")]
        outs.append(read(be, be.where_cond(a, a, b)))
        outs.append(read(be, be.neg(a)))
        outs.append(read(be, be.floor(be.mul(a, b))))       # two roundings: the product, then floor of the fp8 value
        return outs

    def expect():
        with np.errstate(all="ignore"):
            return [f8_round(av + bv), f8_round(av - bv), f8_round(av * bv), f8_round(av / bv),
                    (av < bv).astype(np.float32), (av >= bv).astype(np.float32), (av == bv).astype(np.float32),
                    np.where(av > 0, av, bv), -av, f8_round(np.floor(f8_round(av * bv)))]

    return run, expect


@case("fp8_views_and_gathers")
def _():
    bits, vals = f8_inputs(920, (3, 5, 16), 30.0)
    ids = np.array([4, 0, 2, 2], dtype=np.uint32)

    def run(be):
        t = be.ndarray_from_vec_fp8(bits, bits.shape)
        return [read(be, be.transpose(t, 0, 2)), read(be, be.slice(t, 1, 1, 3)), read(be, be.concat(t, be.neg(t), 2)),
                read(be, be.index(t, 1, be.from_numpy(ids))), read(be, be.broadcast(be.slice(t, 0, 1, 1), (4, 5, 16))),
                read(be, be.max(t)), be.to_numpy(be.argmax(t)), read(be, be.zeros((2, 3), A.F8))]

    def expect():
        return [vals.transpose(2, 1, 0), vals[:, 1:4], np.concatenate([vals, -vals], 2), vals[:, ids],
                np.broadcast_to(vals[1:2], (4, 5, 16)), vals.max(-1, keepdims=True),
                argmax_last(vals), np.zeros((2, 3), np.float32)]

    return run, expect


@case("fp8_transcendental", "ulp_f8")
def _():
    bits, vals = f8_inputs(930, (40, 64), 2.0)
    pos = np.abs(vals) + np.float32(0.25)
    pb = f8_encode(f8_round(pos))
    pv = f8_decode(pb)

    def run(be):
        t, p = be.ndarray_from_vec_fp8(bits, bits.shape), be.ndarray_from_vec_fp8(pb, pb.shape)
        return [read(be, be.exp(t)), read(be, be.sin(t)), read(be, be.cos(t)), read(be, be.log(p)), read(be, be.pow(p, t))]

    def expect():
        v, q = vals.astype(np.float64), pv.astype(np.float64)
        return [f8_round(np.exp(v)), f8_round(np.sin(v)), f8_round(np.cos(v)), f8_round(np.log(q)), f8_round(np.power(q, v))]

    return run, expect


@case("fp8_matmul_sum", "ulp_f8")
def _():
    """f32 accumulation, one rounding at the end (what Candle accumulates in is not restated: parity unpinned)."""
    ab, av = f8_inputs(940, (2, 24, 48), 1.0)
    bb, bv = f8_inputs(941, (2, 48, 40), 1.0)
    sb, sv = f8_inputs(942, (8, 300), 1.0)

    def run(be):
        a, b, s = (be.ndarray_from_vec_fp8(x, x.shape) for x in (ab, bb, sb))
        return [read(be, be.matmul(a, b)), read(be, be.sum(s))]

    def expect():
        return [f8_round(av.astype(np.float64) @ bv.astype(np.float64)), f8_round(sv.astype(np.float64).sum(-1, keepdims=True))]

    return run, expect


@case("fp8_matmul_narrow_operands", "ulp_f8")
def _():
    """A product big enough for the 256 x 256 tile and without a batch axis: the operands are narrowed to their bytes in
    memory and multiplied on the fp8 matrix instructions (k a multiple of 16 but not of the tile depth, ragged edges)."""
    ab, av = f8_inputs(950, (4000, 48), 0.5)
    bb, bv = f8_inputs(951, (4100, 48), 0.5)

    def run(be):
        a, b = be.ndarray_from_vec_fp8(ab, ab.shape), be.ndarray_from_vec_fp8(bb, bb.shape)
        return [read(be, be.matmul(a, be.transpose(b, 0, 1)))]

    def expect():
        p = av.astype(np.float64) @ bv.astype(np.float64).T
        return [f8_round(p)]

    return run, expect


@case("fp8_linear_few_rows_narrow_weights", "ulp_f8")
def _():
    """Decode-time linear layers of fp8 tensors (1 and 4 rows): the weight matrix is narrowed to its bytes in memory once
    and read at one byte a weight."""
    shapes = ((1, 512, 300), (4, 2048, 1024))
    data = []
    for i, (B, K, Nn) in enumerate(shapes):
        ab, av = f8_inputs(960 + i, (B, 1, K), 0.25)
        wb, wv = f8_inputs(970 + i, (Nn, K), 0.25)
        data.append((ab, wb, av, wv))

    def run(be):
        outs = []
        for (B, K, Nn), (ab, wb, _, _) in zip(shapes, data):
            a, w = be.ndarray_from_vec_fp8(ab, ab.shape), be.ndarray_from_vec_fp8(wb, wb.shape)
            outs.append(read(be, be.matmul(a, be.broadcast(be.transpose(w, 0, 1), (B, K, Nn)))))
        return outs

    def expect():
        return [f8_round(av.astype(np.float64) @ wv.astype(np.float64).T) for (_, _, av, wv) in data]

    return run, expect

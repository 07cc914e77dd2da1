"""Cases for the 16-bit float dtypes (f16 = IEEE binary16, bf16 = bfloat16), appended to `cases.CASES`.

NdArrayBackend has `todo!()` for these dtypes (ndarray.rs:7-9); the semantics tested here are those of the
`half` crate that CandleBackend's CPU path rests on (candle.rs:530-551, 575-599, 605-718): widen exactly, compute
in f32, round to nearest even.  What pins them without Candle:
  * conversions and +, -, *, / on f16: numpy's float16 (same model: numpy converts to float32, computes, rounds);
  * bf16 rounding: its closed form on the bit pattern, cross-checked against torch.bfloat16 in test_oracle_half.py;
  * exp/log/sin/cos/pow: float64 evaluation of the exactly held inputs, one unit in the last place of the dtype;
  * matmul / sum (f32 accumulation, one rounding — Candle's accumulation is NOT restated: parity unpinned):
    float64 evaluation, one unit in the last place plus the 1e-3 reduction tolerance.
bf16 tensors cross the test API as uint16 bit patterns (numpy has no bfloat16).
"""
import numpy as np

from catgrad_amd import _abi as A
from cases import CASES, Case, argmax_last, f32, rng, u32


def case(name, kind="exact", scale=None):
    def deco(pair):
        run, expect = pair()
        CASES.append(Case(name, run, expect, kind, scale))
        return pair

    return deco


# ---- bf16 on bit patterns ------------------------------------------------------------------------------------
def bf16_round_bits(x):
    """float32 array -> uint16 bfloat16 bit patterns, round to nearest even; any NaN -> 0x7FC0."""
    x = np.asarray(x, dtype=np.float32)
    u = np.ascontiguousarray(x).reshape(-1).view(np.uint32).astype(np.uint64)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return np.where(nan, 0x7FC0, r).astype(np.uint16).reshape(x.shape)  # NaNs as `read` reports them


def bf16_widen(bits):
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.reshape(-1).astype(np.uint32) << 16).view(np.float32).reshape(bits.shape)


def bf16_values(seed, shape, scale=1.0):
    """Random bf16-representable values as (bits, float32 values)."""
    bits = bf16_round_bits(f32(seed, shape, scale))
    return bits, bf16_widen(bits)


def from_half(be, dt, arr):
    """arr: float16 array (f16) or uint16 bit patterns (bf16)."""
    return be.ndarray_from_vec_f16(arr, arr.shape) if dt == A.F16 else be.ndarray_from_vec_bf16(arr, arr.shape)


def read(be, t):
    """`to_numpy`, with every bf16 NaN mapped to one pattern: which NaN an invalid operation yields (sign,
    payload) differs between processors and is not part of the value."""
    a = be.to_numpy(t)
    if a.dtype == np.uint16:
        a = np.where((a & 0x7FFF) > 0x7F80, np.uint16(0x7FC0), a)
    return a


def as_f32(dt, arr):
    """What `to_numpy` returned for a tensor of dtype dt -> float32 values."""
    return arr.astype(np.float32) if dt == A.F16 else bf16_widen(arr)


def round_to(dt, x):
    """float array -> the dtype's `to_numpy` representation of the rounded values (from float32: one rounding)."""
    x32 = np.asarray(x, dtype=np.float32)
    return x32.astype(np.float16) if dt == A.F16 else bf16_round_bits(x32)


def half_inputs(dt, seed, shape, scale=1.0):
    """(what to upload, float32 values) of random representable numbers."""
    if dt == A.F16:
        h = f32(seed, shape, scale).astype(np.float16)
        return h, h.astype(np.float32)
    return bf16_values(seed, shape, scale)


EDGE_F32 = np.array([0.0, -0.0, 1.0, -1.0, 65504.0, 65519.99, 65520.0, 65536.0, -65520.0, 1e38, 3.4e38, -3.4e38, np.inf, -np.inf,
                     np.nan, 5.9604645e-08, 2.9802322e-08, 2.9802326e-08, 8.940697e-08, 6.097555e-05, 6.1035156e-05, 1e-10,
                     1.0009765625, 1.00048828125, 1.00146484375, 1.0000001, 0.333333, 2049.0, 2051.0, 1.00390625, 1.01171875,
                     3.3895314e38, 3.3961775e38, 1e-40, -1e-45], dtype=np.float32)

NAMES = {A.F16: "f16", A.BF16: "bf16"}

# ---- conversions: from_vec / to_vec / cast matrix --------------------------------------------------------------
for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_all_bit_patterns_roundtrip")
    def _(dt=_dt):
        """Every 16-bit pattern in, the same value out; widening to f32 is exact."""
        bits = np.arange(65536, dtype=np.uint32).astype(np.uint16).reshape(256, 256)
        up = bits.view(np.float16) if dt == A.F16 else bits
        wide = up.astype(np.float32) if dt == A.F16 else bf16_widen(bits)

        def run(be):
            t = from_half(be, dt, up)
            back = read(be, t)
            w = read(be, be.cast(t, A.F32))
            return [np.where(np.isnan(as_f32(dt, back)), 0x7FFF, back.view(np.uint16)), w]

        def expect():
            return [np.where(np.isnan(wide), 0x7FFF, bits), wide]

        return run, expect

    @case(f"half_{NAMES[_dt]}_cast_matrix")
    def _(dt=_dt):
        """f32 -> dtype rounds to nearest even (ties, subnormals, overflow, NaN); dtype -> u32 is Rust `as`
        on the value; u32 -> dtype goes through f32; the other 16-bit dtype rounds again."""
        other = A.BF16 if dt == A.F16 else A.F16
        x = np.concatenate([EDGE_F32, f32(800, (4000,), 50.0), f32(801, (4000,), 1e-6), f32(802, (4000,), 1e4)])
        n = u32(803, (3000,))
        n[:6] = [0, 1, 65519, 65520, 2**24 + 1, 2**32 - 1]
        up, vals = half_inputs(dt, 804, (2000,), 300.0)

        def run(be):
            tx = be.from_numpy(x)
            tn = be.from_numpy(n)
            th = from_half(be, dt, up)
            return [read(be, be.cast(tx, dt)), read(be, be.cast(tn, dt)), read(be, be.cast(th, A.U32)),
                    read(be, be.cast(th, other)), read(be, be.cast(th, A.F32)), read(be, be.cast(th, dt))]

        def expect():
            from cases import rust_f32_as_u32
            with np.errstate(over="ignore"):
                return [round_to(dt, x), round_to(dt, n.astype(np.float32)), rust_f32_as_u32(vals), round_to(other, vals), vals,
                        up]

        return run, expect


# ---- element-wise: exact ops ---------------------------------------------------------------------------------
for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_arithmetic_exact")
    def _(dt=_dt):
        """+, -, *, / computed in f32 and rounded once; comparisons, where, neg, floor, round are exact."""
        ua, a = half_inputs(dt, 810, (33, 130), 8.0)
        ub, b = half_inputs(dt, 811, (33, 130), 8.0)
        b[0, :4] = [0.0, -0.0, np.inf, np.nan]
        a[0, :4] = [1.0, -1.0, np.inf, 2.0]
        a[1, :3] = [60000.0, -60000.0, 1e-7]          # overflow of the sum / product in f16, tiny quotients
        b[1, :3] = [60000.0, 60000.0, 300.0]
        ua, ub = round_to(dt, a), round_to(dt, b)
        a, b = as_f32(dt, ua), as_f32(dt, ub)

        def run(be):
            ta, tb = from_half(be, dt, ua), from_half(be, dt, ub)
            outs = [be.add(ta, tb), be.sub(ta, tb), be.mul(ta, tb), be.div(ta, tb), be.lt(ta, tb), be.gte(ta, tb), be.eq(ta, ta),
                    be.where_cond(be.gt(ta, tb), ta, tb), be.neg(ta), be.floor(ta), be.round(ta),
                    be.add(be.mul(ta, tb), ta)]               # two roundings, not a fused multiply-add
            assert all(o.dtype == dt for o in outs)
            return [read(be, o) for o in outs]

        def expect():
            with np.errstate(all="ignore"):
                one = lambda m: round_to(dt, m.astype(np.float32))
                prod = as_f32(dt, round_to(dt, a * b))
                return [round_to(dt, a + b), round_to(dt, a - b), round_to(dt, a * b), round_to(dt, a / b), one(a < b), one(a >= b),
                        one(a == a), round_to(dt, np.where(a > b, a, b)), round_to(dt, -a), round_to(dt, np.floor(a)),
                        round_to(dt, np.rint(a)), round_to(dt, prod + a)]

        return run, expect

    @case(f"half_{NAMES[_dt]}_scalars_fold_like_tensors")
    def _(dt=_dt):
        """One-element tensors never reach the device: their arithmetic must round the same way."""
        vals = np.array([1.0009765625, 3.0, 0.1, 1e-3, 200.0], dtype=np.float32)
        ups = [round_to(dt, np.array(v, np.float32)) for v in vals]

        def run(be):
            ts = [from_half(be, dt, u.reshape(())) for u in ups]
            outs = []
            for i in range(len(ts) - 1):
                x, y = ts[i], ts[i + 1]
                outs += [be.add(x, y), be.mul(x, y), be.div(x, y), be.sub(x, y), be.cast(be.cast(x, A.F32), dt),
                         be.broadcast(be.div(x, y), (3,))]
            return [read(be, o) for o in outs]

        def expect():
            v = [as_f32(dt, u) for u in ups]
            outs = []
            for i in range(len(v) - 1):
                x, y = v[i], v[i + 1]
                outs += [round_to(dt, x + y), round_to(dt, x * y), round_to(dt, x / y), round_to(dt, x - y), round_to(dt, x),
                         np.broadcast_to(round_to(dt, x / y), (3,))]
            return outs

        return run, expect


# ---- element-wise: libm ops, one unit in the last place --------------------------------------------------------
for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_transcendental", "ulp_" + NAMES[_dt])
    def _(dt=_dt):
        ua, a = half_inputs(dt, 820, (17, 300), 3.0)
        up_, p = half_inputs(dt, 821, (17, 300), 1.5)
        pos = np.abs(a) + np.float32(0.125)
        upos = round_to(dt, pos)
        pos = as_f32(dt, upos)

        def run(be):
            ta, tp, tpos = from_half(be, dt, ua), from_half(be, dt, up_), from_half(be, dt, upos)
            outs = [be.exp(ta), be.sin(ta), be.cos(ta), be.log(tpos), be.pow(tpos, tp)]
            return [as_f32(dt, read(be, o)) for o in outs]

        def expect():
            a64, p64, pos64 = a.astype(np.float64), p.astype(np.float64), pos.astype(np.float64)
            # beyond the dtype's range the rounded result is infinite (halfway between the largest value and 2^emax+1)
            top = 65520.0 if dt == A.F16 else float(np.float32(3.3961775e38))
            inf = lambda v: np.where(np.abs(v) >= top, np.sign(v) * np.inf, v)
            return [inf(np.exp(a64)), np.sin(a64), np.cos(a64), np.log(pos64), inf(pos64 ** p64)]

        return run, expect


# ---- contraction and reductions ---------------------------------------------------------------------------------
def _reduction_inputs(dt):
    ux, x = half_inputs(dt, 830, (3, 40, 96), 1.0)
    uw, w = half_inputs(dt, 831, (3, 96, 72), 1.0)
    ux, uw = round_to(dt, np.abs(x)), round_to(dt, np.abs(w))
    us, s = half_inputs(dt, 832, (5, 7, 333), 4.0)
    s[0, 0, :] = np.nan                                  # max ignores NaN; a row of NaN gives the f32::MIN seed, rounded
    s[1, 2, 5] = s[1, 2, 300] = 1000.0                   # equal maxima: argmax takes the last
    us = round_to(dt, s)
    spos = np.abs(np.nan_to_num(as_f32(dt, us), nan=1.0))
    return ux, uw, us, round_to(dt, spos)


for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_matmul_sum", "ulp_" + NAMES[_dt])
    def _(dt=_dt):
        """f32 accumulation of exactly held values, one rounding (positive data: no cancellation, so one unit in
        the last place of the result covers the accumulation order too)."""
        ux, uw, _us, uspos = _reduction_inputs(dt)
        x, w, spos = as_f32(dt, ux), as_f32(dt, uw), as_f32(dt, uspos)

        def run(be):
            tx, tw, tp = from_half(be, dt, ux), from_half(be, dt, uw), from_half(be, dt, uspos)
            mm = be.matmul(tx, tw)
            mt = be.matmul(be.transpose(tw, 1, 2), be.transpose(tx, 1, 2))     # strided operands
            sm = be.sum(tp)
            assert mm.dtype == dt and sm.dtype == dt
            return [as_f32(dt, read(be, o)) for o in (mm, mt, sm)]

        def expect():
            x64, w64 = x.astype(np.float64), w.astype(np.float64)
            return [x64 @ w64, (x64 @ w64).transpose(0, 2, 1), spos.astype(np.float64).sum(-1, keepdims=True)]

        return run, expect

    @case(f"half_{NAMES[_dt]}_max_argmax_topk")
    def _(dt=_dt):
        _ux, _uw, us, uspos = _reduction_inputs(dt)
        s, spos = as_f32(dt, us), as_f32(dt, uspos)

        def run(be):
            ts, tp = from_half(be, dt, us), from_half(be, dt, uspos)
            mx, am = be.max(ts), be.argmax(ts)
            tv, ti = be.topk(tp, 3)
            assert mx.dtype == dt and am.dtype == A.U32 and tv.dtype == dt and ti.dtype == A.U32
            return [read(be, o) for o in (mx, am, tv, ti)]

        def expect():
            from cases import max_last_f32, topk_ref
            with np.errstate(over="ignore"):
                mx = round_to(dt, max_last_f32(s))
            tv, ti = topk_ref(spos, 3)
            return [mx, argmax_last(s), round_to(dt, tv), ti]

        return run, expect


for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_matmul_mfma_tiles", "ulp_" + NAMES[_dt])
    def _(dt=_dt):
        """Products large enough for the 16-bit matrix instructions in both macro tiles (256 x 256 needs 256 of them),
        all four operand layouts, ragged edges and a k tail that is not a multiple of the tile depth."""
        ux, x = half_inputs(dt, 850, (64, 512, 40), 1.0)
        uw, w = half_inputs(dt, 851, (64, 40, 512), 1.0)
        ux, uw = round_to(dt, np.abs(x)), round_to(dt, np.abs(w))
        x, w = as_f32(dt, ux), as_f32(dt, uw)
        ur, r = half_inputs(dt, 852, (43, 300, 70), 1.0)
        us, s_ = half_inputs(dt, 853, (43, 70, 520), 1.0)
        ur, us = round_to(dt, np.abs(r)), round_to(dt, np.abs(s_))
        r, s_ = as_f32(dt, ur), as_f32(dt, us)

        def run(be):
            tx, tw, tr, ts = (from_half(be, dt, u) for u in (ux, uw, ur, us))
            outs = [be.matmul(tx, tw), be.matmul(tr, ts),
                    be.matmul(be.transpose(ts, 1, 2), be.transpose(tr, 1, 2)),                       # both operands transposed
                    be.matmul(be.slice(tr, 1, 0, 150), ts)]                                          # 128 x 128 tiles
            assert all(o.dtype == dt for o in outs)
            return [as_f32(dt, read(be, o)) for o in outs]

        def expect():
            x64, w64, r64, s64 = (a.astype(np.float64) for a in (x, w, r, s_))
            return [x64 @ w64, r64 @ s64, (r64 @ s64).transpose(0, 2, 1), r64[:, :150] @ s64]

        return run, expect


for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_matmul_narrow_operands", "ulp_" + NAMES[_dt])
    def _(dt=_dt):
        """Products without a batch axis (or with it folded into the rows, as a linear layer's) and enough 256 x 256 tiles
        for a whole device: the operands are narrowed to 2-byte patterns in memory first and multiplied from those.
        Ragged edges, k a multiple of 8 but not of the tile depth, the right operand k-contiguous (a weight matrix
        [out, in] transposed), row-contiguous, and shared by a batch that folds into the rows (the same weight again)."""
        ux, x = half_inputs(dt, 860, (4000, 40), 1.0)
        uw, w = half_inputs(dt, 861, (4100, 40), 1.0)
        ux, uw = round_to(dt, np.abs(x)), round_to(dt, np.abs(w))
        x, w = as_f32(dt, ux), as_f32(dt, uw)
        uy = np.ascontiguousarray(uw.T)

        def run(be):
            tx, tw, ty = (from_half(be, dt, u) for u in (ux, uw, uy))
            x3 = be.reshape(be.slice(tx, 0, 0, 3840), (2, 1920, 40))
            outs = [be.matmul(tx, be.transpose(tw, 0, 1)), be.matmul(tx, ty),
                    be.matmul(x3, be.broadcast(be.transpose(tw, 0, 1), (2, 40, 4100)))]   # the narrowed weight is found again
            assert all(o.dtype == dt for o in outs)
            return [as_f32(dt, read(be, o)) for o in outs]

        def expect():
            p = x.astype(np.float64) @ w.astype(np.float64).T
            return [p, p, p[:3840].reshape(2, 1920, 4100)]

        return run, expect


for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_linear_few_rows_narrow_weights", "ulp_" + NAMES[_dt])
    def _(dt=_dt):
        """Decode-time linear layers of a 16-bit dtype (1, 4 and 8 rows; the batch folds into the rows): the weight matrix
        is narrowed to 2-byte patterns in memory once and read at 2 bytes a weight (up to four rows and K a multiple of 1024:
        the 4 x 4 x 4 matrix-instruction kernel at its four depths, ragged column counts; else a wave per column); the same
        weight used twice."""
        shapes = ((1, 512, 300), (4, 2048, 1024), (8, 1024, 640), (2, 1024, 518), (3, 8192, 262), (4, 4096, 2050))
        data = []
        for i, (B, K, Nn) in enumerate(shapes):
            ux, x = half_inputs(dt, 870 + i, (B, 1, K), 1.0)
            uw, w = half_inputs(dt, 880 + i, (Nn, K), 1.0)
            ux, uw = round_to(dt, np.abs(x)), round_to(dt, np.abs(w))
            data.append((ux, uw, as_f32(dt, ux), as_f32(dt, uw)))

        def run(be):
            outs = []
            for (B, K, Nn), (ux, uw, _, _) in zip(shapes, data):
                tx, tw = from_half(be, dt, ux), from_half(be, dt, uw)
                wv = be.broadcast(be.transpose(tw, 0, 1), (B, K, Nn))
                outs += [be.matmul(tx, wv), be.matmul(be.add(tx, tx), wv)]
            assert all(o.dtype == dt for o in outs)
            return [as_f32(dt, read(be, o)) for o in outs]

        def expect():
            outs = []
            for (_, _, x, w) in data:
                p = x.astype(np.float64) @ w.astype(np.float64).T
                outs += [p, 2.0 * p]
            return outs

        return run, expect


# ---- shape and index ops carry the dtype --------------------------------------------------------------------------
for _dt in (A.F16, A.BF16):
    @case(f"half_{NAMES[_dt]}_views_concat_index")
    def _(dt=_dt):
        ua, a = half_inputs(dt, 840, (4, 6, 10), 2.0)
        ub, _b = half_inputs(dt, 841, (4, 2, 10), 2.0)
        ids = np.array([5, 0, 0, 3], np.uint32)

        def run(be):
            ta, tb = from_half(be, dt, ua), from_half(be, dt, ub)
            outs = [be.transpose(ta, 0, 2), be.slice(ta, 1, 2, 3), be.reshape(ta, (24, 10)), be.broadcast(be.slice(ta, 0, 1, 1), (3, 6, 10)),
                    be.concat(ta, tb, 1), be.index(ta, 1, be.from_numpy(ids)), be.zeros((2, 3), dt),
                    be.concat(be.neg(be.slice(ta, 2, 5, 5)), be.slice(ta, 2, 0, 5), 2)]
            assert all(o.dtype == dt for o in outs)
            return [read(be, o) for o in outs] + [np.array(be.to_bool(ta)), np.array(be.compare(ta, ta))]

        def expect():
            neg = lambda u: round_to(dt, -as_f32(dt, u))
            return [ua.transpose(2, 1, 0), ua[:, 2:5], ua.reshape(24, 10), np.broadcast_to(ua[1:2], (3, 6, 10)),
                    np.concatenate([ua, ub], 1), ua[:, ids], round_to(dt, np.zeros((2, 3), np.float32)),
                    np.concatenate([neg(ua[..., 5:]), ua[..., :5]], 2), np.array(True), np.array(True)]

        return run, expect

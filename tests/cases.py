"""Seeded op cases shared by the CPU suite (oracle vs numpy closed forms) and the GPU
suite (HipBackend vs oracle).

Every case is `Case(name, run, expect, kind)`:
  run(be)   -> list of numpy arrays produced through the Backend API of `be`
  expect()  -> the same list computed by numpy (closed form / float64), or None when
               only backend-vs-backend comparison makes sense
  kind      -> "exact" (bit-exact: integer, shape, index ops and IEEE-exact f32 ops),
               "ew"    (f32 element-wise math: rtol 1e-4, atol 1e-6),
               "ew_abs" (element-wise math fed by a row sum: rtol 1e-4, atol 1e-5),
               "red"   (matmul / sum: 1e-3 of the natural scale of the result)
The tolerances are the ones the north-star states: bit-exact for integer/shape/index
ops, rtol 1e-4 for f32 element-wise, 1e-3 relative for matmul and reductions.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, List, Optional

import numpy as np

from catgrad_amd import _abi as A

F32_MIN = np.float32(-3.4028234663852886e38)


@dataclass
class Case:
    name: str
    run: Callable
    expect: Optional[Callable]
    kind: str = "exact"
    scale: Optional[Callable] = None  # for "red": per-element magnitude bound


def rng(seed):
    return np.random.default_rng(seed)


def f32(seed, shape, scale=1.0):
    return (rng(seed).standard_normal(shape) * scale).astype(np.float32)


def u32(seed, shape, hi=2**32):
    return rng(seed).integers(0, hi, size=shape, dtype=np.uint64).astype(np.uint32)


def total_key(x):
    b = x.astype(np.float32).view(np.int32).astype(np.int64)
    return np.where(b < 0, b ^ 0x7FFFFFFF, b)


def argmax_last(x):
    """Reference rule (ndarray.rs:670-694): max_by(total_cmp) => last of equal maxima."""
    key = total_key(x) if x.dtype == np.float32 else x.astype(np.int64)
    n = key.shape[-1]
    rev = key[..., ::-1]
    return (n - 1 - np.argmax(rev, axis=-1)).astype(np.uint32)[..., None]


def max_last_f32(x):
    """fold from f32::MIN with f32::max: NaN ignored (ndarray.rs:656-661)."""
    y = np.where(np.isnan(x), F32_MIN, x)
    return np.maximum(np.max(y, axis=-1, keepdims=True, initial=F32_MIN), F32_MIN).astype(np.float32)


def rust_f32_as_u32(x):
    x64 = x.astype(np.float64)
    out = np.zeros(x.shape, dtype=np.uint32)
    ok = ~np.isnan(x64)
    clipped = np.clip(np.trunc(np.where(ok, x64, 0.0)), 0.0, 4294967295.0)
    return np.where(ok, clipped, 0).astype(np.uint64).astype(np.uint32)


def wrapping_pow(a, e):
    a = a.astype(np.uint64)
    out = np.ones_like(a)
    e = e.copy()
    M = np.uint64(0xFFFFFFFF)
    for _ in range(32):
        out = np.where(e & 1, (out * a) & M, out)
        a = (a * a) & M
        e = e >> 1
    return out.astype(np.uint32)


def topk_ref(x, k):
    key = total_key(x)
    idx = np.argsort(-key, axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(x, idx, axis=-1), idx.astype(np.uint32)


# ---------------------------------------------------------------------------------------
CASES: List[Case] = []


def case(name, kind="exact", scale=None):
    def deco(pair):
        run, expect = pair()
        CASES.append(Case(name, run, expect, kind, scale))
        return pair

    return deco


def N(be, *ts):
    return [be.to_numpy(t) for t in ts]


# ---- creation ----------------------------------------------------------------------------
for _n in (0, 1, 5, 2304, 70001):
    @case(f"arange_{_n}")
    def _(n=_n):
        return (lambda be: N(be, be.arange(n))), (lambda: [np.arange(n, dtype=np.uint32)])

for _shape in ([], [1], [3, 0, 2], [16, 4, 8, 0, 64], [7, 5]):
    for _dt, _np in ((A.F32, np.float32), (A.U32, np.uint32)):
        @case(f"zeros_{_dt}_{'x'.join(map(str, _shape)) or 'scalar'}")
        def _(shape=_shape, dt=_dt, npdt=_np):
            return (lambda be: N(be, be.zeros(shape, dt))), (lambda: [np.zeros(shape, dtype=npdt)])


@case("from_vec_roundtrip")
def _():
    a, b, s = f32(1, (3, 5, 7)), u32(2, (4, 6)), np.float32(2.5).reshape(())
    return (lambda be: N(be, be.from_numpy(a), be.from_numpy(b), be.from_numpy(s))), (lambda: [a, b, s])


# ---- cast -----------------------------------------------------------------------------------
CAST_F = np.array([0.0, -0.0, 0.9, 1.5, -1.5, 2.9999998, 16777217.0, 4294967040.0, 4294967296.0, 1e20, -1e20,
                   np.nan, np.inf, -np.inf, 1e-40, 3.5e9], dtype=np.float32)
CAST_U = np.array([0, 1, 16777216, 16777217, 16777218, 16777219, 2147483648 + 129, 4294967295, 4294967167,
                   4294967168, 33554435], dtype=np.uint32)


@case("cast_f32_to_u32_rust_as")
def _():
    return (lambda be: N(be, be.cast(be.from_numpy(CAST_F), A.U32))), (lambda: [rust_f32_as_u32(CAST_F)])


@case("cast_u32_to_f32_rne")
def _():
    return (lambda be: N(be, be.cast(be.from_numpy(CAST_U), A.F32))), (lambda: [CAST_U.astype(np.float32)])


@case("cast_identity_and_random")
def _():
    a = f32(3, (33, 17), 1000.0)
    u = u32(4, (129,))
    return (
        lambda be: N(be, be.cast(be.from_numpy(a), A.F32), be.cast(be.from_numpy(a), A.U32),
                     be.cast(be.from_numpy(u), A.U32), be.cast(be.from_numpy(u), A.F32)),
        lambda: [a, rust_f32_as_u32(a), u, u.astype(np.float32)],
    )


# ---- binary -----------------------------------------------------------------------------------
SPECIAL = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, 3.4e38, -3.4e38, 0.5, 2.0], dtype=np.float32)


def _bin_f32(name, npf, kind="exact"):
    @case(f"{name}_f32", kind)
    def _():
        a, b = f32(10, (37, 65)), f32(11, (37, 65))
        sa, sb = np.meshgrid(SPECIAL, SPECIAL)
        sa, sb = np.ascontiguousarray(sa), np.ascontiguousarray(sb)

        def run(be):
            return N(be, getattr(be, name)(be.from_numpy(a), be.from_numpy(b)),
                     getattr(be, name)(be.from_numpy(sa), be.from_numpy(sb)))

        def expect():
            with np.errstate(all="ignore"):
                return [npf(a, b), npf(sa, sb)]

        return run, expect


_bin_f32("add", lambda a, b: a + b)
_bin_f32("sub", lambda a, b: a - b)
_bin_f32("mul", lambda a, b: a * b)
_bin_f32("div", lambda a, b: a / b)
_bin_f32("lt", lambda a, b: (a < b).astype(np.float32))
_bin_f32("gt", lambda a, b: (a > b).astype(np.float32))
_bin_f32("gte", lambda a, b: (a >= b).astype(np.float32))
_bin_f32("lte", lambda a, b: (a <= b).astype(np.float32))
_bin_f32("eq", lambda a, b: (a == b).astype(np.float32))


def _bin_u32(name, npf):
    @case(f"{name}_u32")
    def _():
        a, b = u32(12, (19, 33)), u32(13, (19, 33))
        b[0, :8] = a[0, :8]
        if name == "div":
            b[b == 0] = 7
        if name == "pow":
            a[:, :16] %= 7
            b %= 40

        def run(be):
            return N(be, getattr(be, name)(be.from_numpy(a), be.from_numpy(b)))

        return run, (lambda: [npf(a, b)])


_bin_u32("add", lambda a, b: a + b)
_bin_u32("sub", lambda a, b: a - b)
_bin_u32("mul", lambda a, b: a * b)
_bin_u32("div", lambda a, b: a // b)
_bin_u32("pow", wrapping_pow)
_bin_u32("lt", lambda a, b: (a < b).astype(np.uint32))
_bin_u32("gt", lambda a, b: (a > b).astype(np.uint32))
_bin_u32("gte", lambda a, b: (a >= b).astype(np.uint32))
_bin_u32("lte", lambda a, b: (a <= b).astype(np.uint32))
_bin_u32("eq", lambda a, b: (a == b).astype(np.uint32))


@case("pow_f32", "ew")
def _():
    a = np.abs(f32(14, (41, 23))) + 0.01
    b = f32(15, (41, 23), 2.0)
    th = np.full((32,), 500000.0, np.float32)
    ex = (np.arange(32, dtype=np.float32) * np.float32(2.0 / 64))

    def run(be):
        return N(be, be.pow(be.from_numpy(a), be.from_numpy(b)), be.pow(be.from_numpy(th), be.from_numpy(ex)),
                 be.pow(be.from_numpy(a), be.from_numpy(np.full_like(a, 0.5))))

    def expect():
        return [np.power(a.astype(np.float64), b.astype(np.float64)),
                np.power(th.astype(np.float64), ex.astype(np.float64)), np.sqrt(a.astype(np.float64))]

    return run, expect


@case("pow_f32_special")
def _():
    a = np.array([-8.0, -2.0, 0.0, 2.0, 1.0, -1.0, 4.0], dtype=np.float32)
    b = np.array([1.0 / 3, 0.5, 0.0, 3.0, np.nan, 2.0, 0.5], dtype=np.float32)

    def run(be):
        return N(be, be.pow(be.from_numpy(a), be.from_numpy(b)))

    # negative base with fractional exponent is NaN (Rust powf); exact small powers
    return run, (lambda: [np.array([np.nan, np.nan, 1.0, 8.0, 1.0, 1.0, 2.0], dtype=np.float32)])


# ---- where --------------------------------------------------------------------------------------
@case("where_f32_nan_mask")
def _():
    m = f32(16, (29, 31))
    m[0, :4] = [np.nan, 0.0, -0.0, 1e-45]
    x, y = f32(17, (29, 31)), f32(18, (29, 31))
    return (lambda be: N(be, be.where_cond(be.from_numpy(m), be.from_numpy(x), be.from_numpy(y)))), (
        lambda: [np.where(m > 0, x, y)])


@case("where_u32")
def _():
    m, x, y = u32(19, (64,), 3), u32(20, (64,)), u32(21, (64,))
    return (lambda be: N(be, be.where_cond(be.from_numpy(m), be.from_numpy(x), be.from_numpy(y)))), (
        lambda: [np.where(m != 0, x, y)])


# ---- unary ----------------------------------------------------------------------------------------
@case("neg_floor_round_exact")
def _():
    a = f32(22, (45, 37), 10.0)
    a[0, :8] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 8388608.5, -0.0]
    u = u32(23, (77,))
    u[0] = 0

    def run(be):
        t = be.from_numpy(a)
        return N(be, be.neg(t), be.floor(t), be.round(t), be.neg(be.from_numpy(u)))

    return run, (lambda: [-a, np.floor(a), np.rint(a), (np.uint64(2**32) - u.astype(np.uint64)).astype(np.uint32)])


@case("exp_log_f32", "ew")
def _():
    a = f32(24, (63, 65), 8.0)
    p = np.abs(f32(25, (63, 65), 50.0)) + 1e-6

    def run(be):
        return N(be, be.exp(be.from_numpy(a)), be.log(be.from_numpy(p)))

    return run, (lambda: [np.exp(a.astype(np.float64)), np.log(p.astype(np.float64))])


@case("sin_cos_rope_range", "ew")
def _():
    a = (rng(26).uniform(-2304.0, 2304.0, size=(128, 65))).astype(np.float32)

    def run(be):
        return N(be, be.sin(be.from_numpy(a)), be.cos(be.from_numpy(a)))

    return run, (lambda: [np.sin(a.astype(np.float64)), np.cos(a.astype(np.float64))])


@case("exp_log_special")
def _():
    a = np.array([-np.inf, np.inf, 0.0, -200.0, 100.0], dtype=np.float32)
    lg = np.array([0.0, -1.0, np.inf, 1.0], dtype=np.float32)

    def run(be):
        return N(be, be.exp(be.from_numpy(a)), be.log(be.from_numpy(lg)))

    return run, (lambda: [np.array([0.0, np.inf, 1.0, 0.0, np.inf], np.float32),
                          np.array([-np.inf, np.nan, np.inf, 0.0], np.float32)])


# ---- views: broadcast / reshape / transpose / slice ---------------------------------------------------
@case("broadcast_patterns")
def _():
    s = np.float32(3.25).reshape(())
    col, row = f32(30, (6, 5, 1)), f32(31, (8,))
    w = f32(32, (7, 9))
    kv = f32(33, (2, 3, 1, 5, 4))

    def run(be):
        return N(be, be.broadcast(be.from_numpy(s), (4, 3)), be.broadcast(be.from_numpy(col), (6, 5, 8)),
                 be.broadcast(be.from_numpy(row), (6, 5, 8)),
                 be.broadcast(be.transpose(be.from_numpy(w), 0, 1), (3, 9, 7)),
                 be.broadcast(be.from_numpy(kv), (2, 3, 4, 5, 4)), be.broadcast(be.from_numpy(row), (0, 8)))

    def expect():
        return [np.broadcast_to(s, (4, 3)), np.broadcast_to(col, (6, 5, 8)), np.broadcast_to(row, (6, 5, 8)),
                np.broadcast_to(w.T, (3, 9, 7)), np.broadcast_to(kv, (2, 3, 4, 5, 4)), np.zeros((0, 8), np.float32)]

    return run, expect


@case("reshape_of_views")
def _():
    a = f32(34, (4, 6, 5, 8))
    u = u32(35, (12, 10))

    def run(be):
        t = be.from_numpy(a)
        return N(be,
                 be.reshape(t, (24, 40)),
                 be.reshape(be.transpose(t, 1, 2), (4, 5, 48)),
                 be.reshape(be.slice(t, 3, 2, 4), (4, 6, 20)),
                 be.reshape(be.slice(t, 1, 1, 3), (12, 40)),
                 be.reshape(be.broadcast(be.reshape(be.slice(t, 1, 0, 1), (4, 1, 1, 5, 8)), (4, 1, 3, 5, 8)), (4, 3, 5, 8)),
                 be.reshape(be.reshape(t, (4, 1, 6, 1, 40)), (4, 6, 40)),
                 be.reshape(be.transpose(be.from_numpy(u), 0, 1), (120,)),
                 be.reshape(be.transpose(be.transpose(t, 0, 3), 1, 2), (8 * 5, 6 * 4)))

    def expect():
        return [a.reshape(24, 40), a.transpose(0, 2, 1, 3).reshape(4, 5, 48), a[..., 2:6].reshape(4, 6, 20),
                a[:, 1:4].reshape(12, 40),
                np.broadcast_to(a[:, 0:1].reshape(4, 1, 1, 5, 8), (4, 1, 3, 5, 8)).reshape(4, 3, 5, 8),
                a.reshape(4, 6, 40), u.T.reshape(120), a.transpose(3, 2, 1, 0).reshape(40, 24)]

    return run, expect


@case("repeat_kv_views_through_other_ops")
def _():
    """reshape(broadcast(x)) that merges a stride-0 axis into its neighbour, consumed by everything
    except matmul (which has its own cases)."""
    x = rng(120).integers(-9, 10, size=(2, 3, 1, 5, 8)).astype(np.float32)  # integer-valued: sums are exact
    y = rng(121).integers(-9, 10, size=(2, 12, 5, 8)).astype(np.float32)

    def rep(be):
        return be.reshape(be.broadcast(be.from_numpy(x), (2, 3, 4, 5, 8)), (2, 12, 5, 8))

    def run(be):
        ty = be.from_numpy(y)
        return N(be, rep(be), be.transpose(rep(be), 1, 2), be.slice(rep(be), 1, 2, 7), be.slice(rep(be), 3, 1, 4),
                 be.add(rep(be), ty), be.sum(rep(be)), be.concat(rep(be), ty, 1), be.reshape(rep(be), (24, 40)),
                 be.max(be.transpose(rep(be), 1, 3)), be.broadcast(rep(be), (3, 2, 12, 5, 8)),
                 be.index(rep(be), 1, be.from_numpy(np.array([11, 0, 5], np.uint32))))

    def expect():
        r = np.repeat(x[:, :, 0], 4, axis=1)
        return [r, r.transpose(0, 2, 1, 3), r[:, 2:9], r[..., 1:5], r + y, r.sum(-1, keepdims=True),
                np.concatenate([r, y], 1), r.reshape(24, 40), r.transpose(0, 3, 2, 1).max(-1, keepdims=True),
                np.broadcast_to(r, (3, 2, 12, 5, 8)), r[:, [11, 0, 5]]]

    return run, expect


@case("transpose_slice_chain")
def _():
    a = f32(36, (5, 7, 9))

    def run(be):
        t = be.from_numpy(a)
        return N(be, be.transpose(t, 0, 2), be.transpose(t, 1, 1), be.slice(t, 0, 4, 1), be.slice(t, 2, 9, 0),
                 be.slice(be.transpose(be.slice(t, 1, 2, 4), 1, 2), 1, 3, 5),
                 be.add(be.transpose(t, 0, 1), be.transpose(t, 0, 1)))

    def expect():
        return [a.transpose(2, 1, 0), a, a[4:5], a[:, :, 9:9], a[:, 2:6].transpose(0, 2, 1)[:, 3:8],
                a.transpose(1, 0, 2) * 2]

    return run, expect


@case("elementwise_on_strided_operands")
def _():
    a, b = f32(37, (6, 10, 12)), f32(38, (10, 6, 12))
    g = f32(39, (12,))
    c = f32(40, (6, 10, 1))

    def run(be):
        ta, tb = be.from_numpy(a), be.from_numpy(b)
        return N(be,
                 be.mul(ta, be.transpose(tb, 0, 1)),
                 be.mul(ta, be.broadcast(be.from_numpy(g), (6, 10, 12))),
                 be.div(ta, be.broadcast(be.from_numpy(c), (6, 10, 12))),
                 be.add(be.slice(ta, 2, 0, 6), be.neg(be.slice(ta, 2, 6, 6))),
                 be.sub(be.broadcast(be.from_numpy(np.float32(1.5).reshape(())), (6, 10, 12)), ta),
                 be.exp(be.transpose(be.slice(ta, 1, 1, 8), 0, 2)))

    def expect():
        return [a * b.transpose(1, 0, 2), a * g, a / c, a[..., :6] + (-a[..., 6:]), np.float32(1.5) - a,
                np.exp(a[:, 1:9].transpose(2, 1, 0).astype(np.float64))]

    return run, expect


CASES[-1].kind = "ew"


# ---- concat / index -------------------------------------------------------------------------------------
@case("concat_all_dims")
def _():
    a, b0, b1, b2 = f32(41, (3, 4, 5)), f32(42, (2, 4, 5)), f32(43, (3, 6, 5)), f32(44, (3, 4, 1))
    e = np.zeros((3, 0, 5), np.float32)
    u1, u2 = u32(45, (4, 3)), u32(46, (4, 2))

    def run(be):
        ta = be.from_numpy(a)
        return N(be, be.concat(ta, be.from_numpy(b0), 0), be.concat(ta, be.from_numpy(b1), 1),
                 be.concat(ta, be.from_numpy(b2), 2), be.concat(be.from_numpy(e), ta, 1),
                 be.concat(ta, be.from_numpy(e), 1), be.concat(be.from_numpy(u1), be.from_numpy(u2), 1),
                 be.concat(be.neg(be.slice(ta, 2, 3, 2)), be.slice(ta, 2, 0, 3), 2),
                 be.concat(be.transpose(ta, 0, 1), be.transpose(ta, 0, 1), 2))

    def expect():
        return [np.concatenate([a, b0], 0), np.concatenate([a, b1], 1), np.concatenate([a, b2], 2), a, a,
                np.concatenate([u1, u2], 1), np.concatenate([-a[..., 3:], a[..., :3]], 2),
                np.concatenate([a.transpose(1, 0, 2)] * 2, 2)]

    return run, expect


@case("kv_restack_chain")
def _():
    layers = [f32(50 + i, (2, 3, 4, 8)) for i in range(5)]

    def run(be):
        out = be.reshape(be.from_numpy(layers[0]), (1, 2, 3, 4, 8))
        for l in layers[1:]:
            out = be.concat(out, be.reshape(be.from_numpy(l), (1, 2, 3, 4, 8)), 0)
        return N(be, out)

    return run, (lambda: [np.stack(layers)])


@case("kv_restack_chain_moved_operands")
def _():
    """Same chain with the growing stack MOVED into every concat, as the interpreter does:
    uniquely owned stacks may be appended to in place."""
    layers = [f32(70 + i, (2, 3, 4, 8)) for i in range(9)]

    def run(be):
        out = be.reshape(be.from_numpy(layers[0]).move(), (1, 2, 3, 4, 8))
        keep = None
        for n, l in enumerate(layers[1:]):
            out = be.concat(out.move(), be.reshape(be.from_numpy(l).move(), (1, 2, 3, 4, 8)).move(), 0)
            if n == 3:
                keep = out.clone()  # a second holder: the next append must not disturb it
        flat = be.concat(be.from_numpy(layers[0].reshape(-1)).move(), be.from_numpy(layers[1].reshape(-1)).move(), 0)
        flat = be.concat(flat.move(), be.from_numpy(layers[2].reshape(-1)).move(), 0)
        return N(be, out, keep, flat)

    return run, (lambda: [np.stack(layers), np.stack(layers[:5]),
                          np.concatenate([l.reshape(-1) for l in layers[:3]])])


@case("kv_cache_growth_loop")
def _():
    """The KV-cache dance of helpers/cache.rs over several steps: per-layer slice + squeeze of the stacked
    cache, concat of new rows along the sequence axis, restack along axis 0 — with operands moved as the
    interpreter does.  Also: an earlier cache stays valid, and two different appends to the same base agree
    with numpy (the second one must not see the first one's rows)."""
    L, B, H, T0, D = 3, 2, 2, 64, 64
    base = f32(130, (L, B, H, T0, D))
    news = [[f32(131 + 10 * s + l, (B, H, 1 + (s % 2), D)) for l in range(L)] for s in range(6)]
    fork = f32(199, (B, H, 2, D))

    def run(be):
        cache = be.from_numpy(base)
        old = []
        forked = None
        for s in range(6):
            layers = []
            for l in range(L):
                c = be.reshape(be.slice(cache, 0, l, 1).move(), (B, H, cache.shape[3], D))
                if s == 2 and l == 1:
                    forked = be.concat(c, be.from_numpy(fork).move(), 2)  # c borrowed: a second append follows
                layers.append(be.concat(c.move(), be.from_numpy(news[s][l]).move(), 2))
            shp = (1, B, H, layers[0].shape[2], D)
            out = be.reshape(layers[0].move(), shp)
            for l in range(1, L):
                out = be.concat(out.move(), be.reshape(layers[l].move(), shp).move(), 0)
            if s in (0, 3):
                old.append(cache.clone())
            cache = out
        return N(be, cache, forked, *old)

    def expect():
        c = base
        olds, forked = [], None
        for s in range(6):
            if s == 2:
                forked = np.concatenate([c[1], fork], 2)
            if s in (0, 3):
                olds.append(c)
            c = np.stack([np.concatenate([c[l], news[s][l]], 2) for l in range(L)])
        return [c, forked, *olds]

    return run, expect


@case("kv_deferred_row_writes", "red")
def _():
    """Rows appended to a cache from element-wise programs (as the rotary embedding of k is) may be written
    late, together with their neighbours: every kind of reader that follows must still see them — read-back,
    a reduction, a gather, a matrix product, another program, a clone taken before the next append — also with
    more appends in a row than one launch takes, and with a deferred left operand of a product joining them."""
    B, H, T0, D = 2, 2, 40, 64
    base = np.abs(f32(700, (B, H, T0, D)))
    rows = [np.abs(f32(701 + i, (B, H, 1, D))) for i in range(7)]
    q = np.abs(f32(720, (B, H, 1, D)))
    ids = np.array([0, T0 + 2, T0 + 6, 5], np.uint32)

    def run(be):
        two = lambda: _const(be, 2.0, (B, H, 1, D))
        cache = be.from_numpy(base)
        outs = []
        for i, r in enumerate(rows):
            new = be.mul(be.from_numpy(r).move(), two().move())        # a deferred program
            cache = be.concat(cache.move(), new.move(), 2)
            if i == 0:
                outs.append(be.to_numpy(cache))                          # read-back right after one append
            if i == 1:
                outs.append(be.to_numpy(be.sum(be.transpose(cache, 2, 3))))   # reduction over the time axis
            if i == 2:
                old = cache.clone()
        outs.append(be.to_numpy(be.index(cache, 2, be.from_numpy(ids))))      # 4 appends waiting: gather
        tq = be.mul(be.from_numpy(q).move(), two().move())                   # deferred left operand
        new = be.add(be.from_numpy(rows[0]).move(), two().move())
        cache = be.concat(cache.move(), new.move(), 2)
        scores = be.matmul(tq.move(), be.transpose(cache, 2, 3).move())      # joins the waiting write
        outs.append(be.to_numpy(scores))
        outs.append(be.to_numpy(be.exp(be.neg(be.slice(cache, 2, T0, 8)))))
        outs.append(be.to_numpy(old))
        outs.append(be.to_numpy(cache))
        return outs

    def expect():
        full = np.concatenate([base] + [2 * r for r in rows] + [rows[0] + 2], 2).astype(np.float64)
        return [full[:, :, :T0 + 1], full[:, :, :T0 + 2].sum(2)[..., None], full[:, :, ids],
                (2 * q.astype(np.float64)) @ full.transpose(0, 1, 3, 2), np.exp(-full[:, :, T0:T0 + 8]),
                full[:, :, :T0 + 3], full]

    return run, expect


@case("constant_programs_are_kept", "ew_abs")
def _():
    """Tables built from iota and scalars (rope.rs:65-104 does this on every forward pass) are computed once
    and handed out again: the second build must equal the first, a different scalar must give different
    values, growing a kept table by concat must not change what the next build sees, and every arange is
    a view of one growing iota.  (Angles up to 100: one ulp of the angle is 8e-6, inside the absolute tolerance.)"""
    n, h = 100, 16

    def table(be, theta, fn):
        pos = be.cast(be.arange(n), A.F32)
        inv = be.pow(_const(be, theta, (h,)), be.neg(be.div(be.cast(be.arange(h), A.F32), _const(be, float(h), (h,)))))
        ang = be.mul(be.broadcast(be.reshape(pos, (n, 1)), (n, h)), be.broadcast(be.reshape(inv, (1, h)), (n, h)))
        half = fn(ang)
        return be.concat(half, half, 1)

    def run(be):
        outs = [be.to_numpy(be.arange(5)), be.to_numpy(be.arange(5000)), be.to_numpy(be.arange(7))]
        t1 = table(be, 100.0, be.cos)
        outs.append(be.to_numpy(t1))
        grown = be.concat(t1.move(), be.from_numpy(np.ones((2, 2 * h), np.float32)).move(), 0)
        outs.append(be.to_numpy(grown))
        outs.append(be.to_numpy(table(be, 100.0, be.cos)))      # kept
        outs.append(be.to_numpy(table(be, 50.0, be.cos)))       # another constant: not the kept one
        outs.append(be.to_numpy(table(be, 100.0, be.sin)))
        return outs

    def expect():
        def tab(theta, fn):
            # the angles as f32 computes them (each step rounded), the function itself in float64
            inv = (np.float64(theta) ** (-(np.arange(h, dtype=np.float32) / np.float32(h)).astype(np.float64))).astype(np.float32)
            ang = (np.arange(n, dtype=np.float32)[:, None] * inv[None, :]).astype(np.float64)
            return np.concatenate([fn(ang), fn(ang)], 1)
        t = tab(100.0, np.cos)
        return [np.arange(5, dtype=np.uint32), np.arange(5000, dtype=np.uint32), np.arange(7, dtype=np.uint32),
                t, np.concatenate([t, np.ones((2, 2 * h))], 0), t, tab(50.0, np.cos), tab(100.0, np.sin)]

    return run, expect


@case("concat_adjacent_views_merge")
def _():
    a = f32(140, (6, 4, 10))

    def run(be):
        t = be.from_numpy(a)
        return N(be, be.concat(be.slice(t, 0, 0, 2), be.slice(t, 0, 2, 3), 0),
                 be.concat(be.slice(t, 2, 1, 4), be.slice(t, 2, 5, 5), 2),
                 be.concat(be.slice(t, 1, 0, 1), be.slice(t, 1, 1, 1), 1),
                 be.concat(be.slice(t, 0, 1, 2), be.slice(t, 0, 4, 2), 0),   # not adjacent: must copy
                 be.concat(be.slice(t, 2, 0, 5), be.slice(t, 2, 0, 5), 2))   # same view twice

    def expect():
        return [a[0:5], a[:, :, 1:10], a[:, 0:2], np.concatenate([a[1:3], a[4:6]], 0),
                np.concatenate([a[..., :5], a[..., :5]], 2)]

    return run, expect


@case("index_gather")
def _():
    w = f32(60, (50, 16))
    ids = u32(61, (23,), 50)
    ids[:3] = [49, 0, 49]
    x3 = u32(62, (4, 6, 5))
    i1, i2 = np.array([5, 0, 0, 3], np.uint32), np.array([4, 4, 1], np.uint32)

    def run(be):
        tw, tx = be.from_numpy(w), be.from_numpy(x3)
        return N(be, be.index(tw, 0, be.from_numpy(ids)), be.index(tx, 1, be.from_numpy(i1)),
                 be.index(tx, 2, be.from_numpy(i2)), be.index(be.transpose(tw, 0, 1), 1, be.from_numpy(ids)),
                 be.index(tw, 0, be.from_numpy(np.zeros((0,), np.uint32))),
                 be.index(tw, 0, be.slice(be.from_numpy(ids), 0, 3, 7)))

    def expect():
        return [w[ids], x3[:, i1], x3[:, :, i2], w.T[:, ids], np.zeros((0, 16), np.float32), w[ids[3:10]]]

    return run, expect


# ---- reductions ---------------------------------------------------------------------------------------------
@case("max_rules")
def _():
    a = f32(70, (9, 130))
    a[0, :] = np.nan
    a[1, :] = -np.inf
    a[2, 5] = np.nan
    a[3, 7] = np.inf
    u = u32(71, (5, 67))
    one = f32(72, (6,))
    e = np.zeros((3, 0), np.float32)

    def run(be):
        return N(be, be.max(be.from_numpy(a)), be.max(be.from_numpy(u)), be.max(be.from_numpy(one)),
                 be.max(be.from_numpy(e)), be.max(be.transpose(be.from_numpy(a), 0, 1)))

    def expect():
        return [max_last_f32(a), u.max(axis=-1, keepdims=True), max_last_f32(one), np.full((3, 1), F32_MIN),
                max_last_f32(a.T)]

    return run, expect


@case("argmax_rules")
def _():
    a = f32(73, (11, 257))
    a[0, :] = 1.0  # all tied -> last index
    a[1, 3] = a[1, 200] = 99.0
    a[2, :] = -0.0
    a[2, 17] = 0.0  # +0 beats -0
    a[3, 40] = np.nan  # +NaN is the greatest
    a[4, 9] = np.inf
    a[5, :] = -np.inf
    neg_nan = np.array([0xFFC00000], dtype=np.uint32).view(np.float32)[0]
    a[6, 100] = neg_nan  # -NaN is the least
    u = u32(74, (6, 33), 5)
    big = f32(75, (2, 128256), 0.02)

    def run(be):
        return N(be, be.argmax(be.from_numpy(a)), be.argmax(be.from_numpy(u)), be.argmax(be.from_numpy(big)),
                 be.argmax(be.slice(be.transpose(be.from_numpy(a), 0, 1), 0, 10, 100)))

    def expect():
        return [argmax_last(a), argmax_last(u), argmax_last(big), argmax_last(np.ascontiguousarray(a.T[10:110]))]

    return run, expect


@case("sum_u32_and_small_f32")
def _():
    u = u32(76, (7, 300))
    ints = rng(77).integers(-8, 9, size=(5, 4, 100)).astype(np.float32)  # exact in any order
    e = np.zeros((4, 0), np.float32)

    def run(be):
        return N(be, be.sum(be.from_numpy(u)), be.sum(be.from_numpy(ints)), be.sum(be.from_numpy(e)),
                 be.sum(be.transpose(be.from_numpy(ints), 1, 2)), be.sum(be.from_numpy(ints[0, 0])))

    def expect():
        return [u.sum(axis=-1, keepdims=True, dtype=np.uint32), ints.sum(-1, keepdims=True), np.zeros((4, 1), np.float32),
                ints.transpose(0, 2, 1).sum(-1, keepdims=True), ints[0, 0].sum(keepdims=True)]

    return run, expect


def _sum_scale(arrs):
    return lambda: [np.abs(a.astype(np.float64)).sum(-1, keepdims=True) for a in arrs]


_SUM_IN = [f32(78, (33, 2048)), f32(79, (3, 5, 77)), np.square(f32(80, (16, 576)))]


@case("sum_f32", "red", _sum_scale(_SUM_IN))
def _():
    def run(be):
        return N(be, *[be.sum(be.from_numpy(a)) for a in _SUM_IN])

    return run, (lambda: [a.astype(np.float64).sum(-1, keepdims=True) for a in _SUM_IN])


@case("topk_rules")
def _():
    a = f32(81, (6, 40))
    a[0, :] = 2.0
    a[1, 5] = a[1, 30] = 50.0
    big = f32(82, (3, 4, 128))

    def run(be):
        v1, i1 = be.topk(be.from_numpy(a), 4)
        v2, i2 = be.topk(be.from_numpy(big), 8)
        v3, i3 = be.topk(be.from_numpy(a), 40)
        return N(be, v1, i1, v2, i2, v3, i3)

    def expect():
        return [*topk_ref(a, 4), *topk_ref(big, 8), *topk_ref(a, 40)]

    return run, expect


# ---- matmul ---------------------------------------------------------------------------------------------------
def _mm_case(name, ashape, bshape, prep=None, seed=90):
    a, b = f32(seed, ashape), f32(seed + 1, bshape)
    prep = prep or (lambda be, ta, tb: (ta, tb, a, b))

    def build(be):
        ta, tb = be.from_numpy(a), be.from_numpy(b)
        return prep(be, ta, tb)

    def run(be):
        x, y, _, _ = build(be)
        return N(be, be.matmul(x, y))

    def views():
        class NP:  # numpy stand-in for the few view ops `prep` uses
            @staticmethod
            def transpose(t, i, j):
                return np.swapaxes(t, i, j)

            @staticmethod
            def broadcast(t, s):
                return np.broadcast_to(t, s)

            @staticmethod
            def reshape(t, s):
                return t.reshape(s)

            @staticmethod
            def slice(t, d, s, l):
                ix = [slice(None)] * t.ndim
                ix[d] = slice(s, s + l)
                return t[tuple(ix)]

        x, y, _, _ = prep(NP, a, b)
        return x.astype(np.float64), y.astype(np.float64)

    def expect():
        x, y = views()
        return [x @ y]

    def scale():
        x, y = views()
        return [np.abs(x) @ np.abs(y)]

    CASES.append(Case(name, run, expect, "red", scale))


_mm_case("mm_2d", (70, 50), (50, 90))
_mm_case("mm_batched_3d", (5, 33, 65), (5, 65, 17))
_mm_case("mm_two_batch_dims", (2, 3, 40, 24), (2, 3, 24, 56))
_mm_case("mm_k1_and_m1", (4, 1, 1), (4, 1, 9))
_mm_case("mm_decode_gemv", (4, 1, 576), (4, 576, 300))
_mm_case("mm_linear_weight_view", (3, 20, 64), (48, 64),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (3, 64, 48)), None, None))
_mm_case("mm_linear_decode", (4, 1, 256), (1000, 256),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (4, 256, 1000)), None, None))
_mm_case("mm_linear_decode_wide_split", (4, 1, 2048), (512, 2048),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (4, 2048, 512)), None, None))
_mm_case("mm_linear_decode_wide_cols1", (4, 1, 512), (5003, 512),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (4, 512, 5003)), None, None))
_mm_case("mm_linear_decode_wide_cols4", (3, 1, 384), (20001, 384),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (3, 384, 20001)), None, None))
_mm_case("mm_linear_decode_mfma_4x4", (4, 1, 388), (8201, 388),   # ragged N and K: clamped rows, zero-filled k tail
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (4, 388, 8201)), None, None))
_mm_case("mm_linear_decode_mfma_4x4_m3_k2304", (3, 1, 2304), (8192, 2304),   # two k chunks, M < 4
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (3, 2304, 8192)), None, None))
_mm_case("mm_linear_m8", (8, 1, 1024), (300, 1024),
         lambda be, x, w: (x, be.broadcast(be.transpose(w, 0, 1), (8, 1024, 300)), None, None))
_mm_case("mm_decode_scores_hd64", (2, 1, 6, 64), (2, 6, 301, 64),
         lambda be, q, k: (be.transpose(q, 1, 2), be.transpose(k, 2, 3), None, None))
_mm_case("mm_decode_scores_hd128", (2, 1, 4, 128), (2, 4, 77, 128),
         lambda be, q, k: (be.transpose(q, 1, 2), be.transpose(k, 2, 3), None, None))
_mm_case("mm_decode_context", (2, 6, 1, 301), (2, 6, 301, 64))
_mm_case("mm_decode_context_ragged_n", (3, 5, 2, 90), (3, 5, 90, 70))
_mm_case("mm_attention_scores", (2, 40, 6, 32), (2, 56, 6, 32),
         lambda be, q, k: (be.transpose(q, 1, 2), be.transpose(be.transpose(k, 1, 2), 2, 3), None, None))
_mm_case("mm_attention_context", (2, 6, 40, 56), (2, 56, 6, 32),
         lambda be, p, v: (p, be.transpose(v, 1, 2), None, None))
_mm_case("mm_repeat_kv_rhs", (2, 6, 5, 16), (2, 2, 1, 16, 12),
         lambda be, q, kv: (q, be.reshape(be.broadcast(kv, (2, 2, 3, 16, 12)), (2, 6, 16, 12)), None, None))
_mm_case("mm_repeat_kv_transposed_rhs", (2, 6, 5, 16), (2, 2, 1, 12, 16),
         lambda be, q, kv: (q, be.transpose(be.reshape(be.broadcast(kv, (2, 2, 3, 12, 16)), (2, 6, 12, 16)), 2, 3),
                            None, None))
_mm_case("mm_repeat_kv_both_operands", (2, 2, 1, 5, 16), (2, 2, 1, 16, 12),
         lambda be, q, kv: (be.reshape(be.broadcast(q, (2, 2, 3, 5, 16)), (2, 6, 5, 16)),
                            be.reshape(be.broadcast(kv, (2, 2, 3, 16, 12)), (2, 6, 16, 12)), None, None))
_mm_case("mm_transposed_lhs", (3, 64, 30), (3, 64, 20), lambda be, a, b: (be.transpose(a, 1, 2), b, None, None))
_mm_case("mm_sliced_operands", (2, 50, 80), (2, 80, 70),
         lambda be, a, b: (be.slice(a, 2, 8, 64), be.slice(be.slice(b, 1, 8, 64), 2, 3, 33), None, None))
_mm_case("mm_k_over_256", (2, 16, 700), (2, 700, 24))
_mm_case("mm_tile_edges", (1, 129, 67), (1, 67, 131))
_mm_case("mm_big_tile", (2, 256, 128), (2, 128, 384))
# enough 256 x 256 tiles to cover the chip: the one-wave-per-SIMD tile, in all four operand layouts, full and ragged
_mm_case("mm_256_tiles_full", (64, 512, 40), (64, 40, 512), seed=96)
_mm_case("mm_256_tiles_ragged", (43, 300, 70), (43, 70, 520), seed=97)
_mm_case("mm_256_tiles_lhs_transposed", (43, 70, 300), (43, 70, 520),
         lambda be, a, b: (be.transpose(a, 1, 2), b, None, None), seed=98)
_mm_case("mm_256_tiles_rhs_transposed", (43, 300, 70), (43, 520, 70),
         lambda be, a, b: (a, be.transpose(b, 1, 2), None, None), seed=99)
_mm_case("mm_256_tiles_both_transposed_linear", (300, 16, 68), (5000, 68),
         lambda be, a, b: (be.transpose(a, 0, 1), be.broadcast(be.transpose(b, 0, 1), (16, 68, 5000)), None, None), seed=100)

# products with fewer 128-wide tiles than compute units (the linear layers of a short prefill on a narrow model): cut
# along k over grid.z, the partial tiles summed in a fixed order.  The linear layers of the Qwen3-0.6B shape at 1024
# positions and of the SmolLM2-135M shape at 512, a k that is no multiple of the tile depth, a row-contiguous right
# operand, a transposed left operand, several batch entries.
def _linear_prep(n_out):
    return lambda be, a, b: (a, be.broadcast(be.transpose(b, 0, 1), (a.shape[0], b.shape[1], n_out)), None, None)


_mm_case("mm_split_k_1024x1024x3072", (1, 1024, 3072), (1024, 3072), _linear_prep(1024), seed=110)
_mm_case("mm_split_k_1024x2048x1024", (1, 1024, 1024), (2048, 1024), _linear_prep(2048), seed=112)
_mm_case("mm_split_k_512x576x576", (1, 512, 576), (576, 576), _linear_prep(576), seed=114)
_mm_case("mm_split_k_512x1536x576", (1, 512, 576), (1536, 576), _linear_prep(1536), seed=116)
_mm_case("mm_split_k_512x576x1536", (1, 512, 1536), (576, 1536), _linear_prep(576), seed=118)
_mm_case("mm_split_k_ragged_k", (1, 300, 1000), (200, 1000), _linear_prep(200), seed=120)
_mm_case("mm_split_k_rhs_rows", (1, 256, 2048), (1, 2048, 384), seed=122)
_mm_case("mm_split_k_lhs_transposed", (2, 1100, 130), (2, 1100, 260), lambda be, a, b: (be.transpose(a, 1, 2), b, None, None), seed=124)
_mm_case("mm_split_k_batched", (3, 128, 1024), (3, 1024, 128), seed=126)


@case("mm_u32_wrapping")
def _():
    a, b = u32(95, (2, 5, 7)), u32(96, (2, 7, 3))

    def run(be):
        return N(be, be.matmul(be.from_numpy(a), be.from_numpy(b)))

    def expect():
        return [(a.astype(np.uint64)[..., :, :, None] * b.astype(np.uint64)[..., None, :, :]).sum(-2).astype(np.uint32)]

    return run, expect


@case("mm_zero_extents")
def _():
    def run(be):
        return N(be, be.matmul(be.zeros((2, 0, 4), A.F32), be.zeros((2, 4, 3), A.F32)),
                 be.matmul(be.from_numpy(f32(97, (2, 3, 0))), be.from_numpy(f32(98, (2, 0, 5)))))

    return run, (lambda: [np.zeros((2, 0, 3), np.float32), np.zeros((2, 3, 5), np.float32)])


# ---- host read-backs ------------------------------------------------------------------------------------------------
@case("to_bool_and_compare")
def _():
    a = f32(99, (13, 7))

    def run(be):
        t = be.from_numpy(a)
        z = be.zeros((4, 4), A.F32)
        nanv = be.from_numpy(np.array([np.nan, -1.0, 0.0], np.float32))
        res = [be.to_bool(t), be.to_bool(z), be.to_bool(nanv), be.to_bool(be.from_numpy(np.array([0, 0, 2], np.uint32))),
               be.to_bool(be.zeros((3,), A.U32)), be.to_bool(be.from_numpy(np.float32(5.0).reshape(()))),
               be.compare(t, be.from_numpy(a)), be.compare(t, be.from_numpy(a + 1)),
               be.compare(be.transpose(t, 0, 1), be.from_numpy(np.ascontiguousarray(a.T))),
               be.compare(t, be.reshape(t, (7, 13))), be.compare(nanv, nanv), be.compare(z, be.zeros((4, 4), A.F32))]
        return [np.array(res, dtype=np.uint32)]

    return run, (lambda: [np.array([1, 0, 0, 1, 0, 1, 1, 0, 1, 0, 0, 1], np.uint32)])


# ---- composites (stdlib definitions) vs float64 formulas -------------------------------------------------------------
def softmax_ops(be, x):
    """`nn::softmax` (catgrad/src/stdlib/nn/mod.rs:168-179) as backend calls."""
    shp = x.shape
    m = be.broadcast(be.max(x), shp)
    ex = be.exp(be.sub(x, m))
    s = be.broadcast(be.sum(ex), shp)
    return be.div(ex, s)


@case("softmax_with_f32_min_entry", "ew")
def _():
    a = f32(100, (7, 96), 3.0)
    a[0, 5] = F32_MIN  # masked entry as built by causal_mask (helpers/tensors.rs:207-224)

    def run(be):
        y = softmax_ops(be, be.from_numpy(a))
        return N(be, y, be.sum(y))

    def expect():
        x = a.astype(np.float64)
        e = np.exp(x - x.max(-1, keepdims=True))
        p = e / e.sum(-1, keepdims=True)
        return [p, np.ones((7, 1))]

    return run, expect


# ---- concat along the last axis stays deferred (piecewise leaf) --------------------------------------------
def _rot_half(be, t, h):
    """helpers/rope.rs:423-427: concat(-x[..., h:], x[..., :h])."""
    nd = len(t.shape) - 1
    return be.concat(be.neg(be.slice(t, nd, h, h)), be.slice(t, nd, 0, h), nd)


for _h, _shape in ((32, (2, 4, 3, 64)), (5, (3, 2, 10)), (8, (4, 16)), (1, (7, 2))):
    @case(f"concat_last_rotate_half_h{_h}")
    def _(h=_h, shape=_shape):
        x = f32(300 + h, shape)
        c = f32(301 + h, shape)
        s_ = f32(302 + h, shape)

        def run(be):
            tx, tc, ts = be.from_numpy(x), be.from_numpy(c), be.from_numpy(s_)
            rot = _rot_half(be, tx, h)
            rope = be.add(be.mul(tc, tx), be.mul(ts, _rot_half(be, tx, h)))   # apply_rope_embedding
            return N(be, rot, rope, be.max(_rot_half(be, tx, h)))

        def expect():
            r = np.concatenate([-x[..., h:], x[..., :h]], -1)
            return [r, c * x + s_ * r, r.max(-1, keepdims=True)]

        return run, expect


@case("concat_last_deferred_variants")
def _():
    """Strided operands, u32, negation on either side, two piecewise operands in one op, views and
    further concats of a deferred concat, uneven parts."""
    a = rng(310).integers(-9, 10, size=(3, 6, 4)).astype(np.float32)
    b = rng(311).integers(-9, 10, size=(3, 6, 7)).astype(np.float32)
    u = u32(312, (5, 3))
    v = u32(313, (5, 8))

    def run(be):
        ta, tb, tu, tv = be.from_numpy(a), be.from_numpy(b), be.from_numpy(u), be.from_numpy(v)
        at = be.transpose(be.from_numpy(a.transpose(1, 0, 2).copy()), 0, 1)      # strided view equal to a
        c1 = be.concat(at, be.neg(tb), 2)
        c2 = be.concat(be.neg(ta), be.neg(tb), 2)
        two = be.add(be.concat(ta, tb, 2), be.concat(be.neg(ta), tb, 2))         # two piecewise operands
        cu = be.add(be.concat(tu, tv, 1), be.concat(tu, tv, 1))
        tr = be.transpose(be.concat(ta, tb, 2), 1, 2)                            # a view ends the deferral
        cc = be.concat(be.concat(ta, tb, 2), ta, 2)                              # deferred concat as an operand
        sl = be.slice(be.concat(ta, tb, 2), 2, 2, 6)
        sm = be.sum(be.mul(be.concat(ta, tb, 2), be.concat(ta, tb, 2)))
        shared = be.concat(ta, tb, 2)
        sh = be.sub(be.mul(shared, shared), shared)
        return N(be, c1, c2, two, cu, tr, cc, sl, sm, sh)

    def expect():
        ab = np.concatenate([a, b], 2)
        uv = np.concatenate([u, v], 1)
        return [np.concatenate([a, -b], 2), np.concatenate([-a, -b], 2), ab + np.concatenate([-a, b], 2), uv + uv,
                ab.transpose(0, 2, 1), np.concatenate([ab, a], 2), ab[:, :, 2:8], (ab * ab).sum(-1, keepdims=True),
                ab * ab - ab]

    return run, expect


# ---- few long rows: segmented reductions --------------------------------------------------------------------
for _shape in ((4, 128256), (3, 70001), (1, 1, 32768), (2, 40000)):
    @case(f"long_rows_argmax_max_sum_{'x'.join(map(str, _shape))}")
    def _(shape=_shape):
        n = shape[-1]
        a = rng(600 + n).integers(-50, 50, size=shape).astype(np.float32)     # integer-valued: sums are exact
        a[..., 5] = 77.0
        a[..., n // 2] = 77.0          # equal maxima in different segments: the last one wins
        a[..., n - 3] = 77.0
        a[0, ..., n - 3] = -1.0
        u = u32(601 + n, shape, hi=1000)

        def run(be):
            t, tu = be.from_numpy(a), be.from_numpy(u)
            return N(be, be.argmax(t), be.max(t), be.sum(t), be.argmax(tu), be.sum(tu),
                     be.argmax(be.add(t, t)))      # a deferred program in front of the reduction

        def expect():
            return [argmax_last(a), a.max(-1, keepdims=True), a.sum(-1, keepdims=True, dtype=np.float64), argmax_last(u),
                    u.astype(np.uint64).sum(-1, keepdims=True).astype(np.uint32), argmax_last(a + a)]

        return run, expect


# ---- copies that transpose, reductions over an axis that is not the unit-stride one ------------------------------------
@case("transpose_copies_tiled")
def _():
    """Row-major copies of transposed views (`reshape` after `transpose`, ndarray.rs:545-569): whole 64 x 64 tiles with
    16-byte accesses, ragged edges, further axes, an unaligned (sliced) source, u32, the head merge of attention."""
    a = f32(600, (130, 70))
    b = u32(601, (256, 512))
    c = f32(602, (257, 513))
    d = f32(603, (4, 6, 64, 128))
    e = f32(604, (3, 200, 96))
    g = f32(605, (128, 260))

    def run(be):
        outs = [be.reshape(be.transpose(be.from_numpy(a), 0, 1), (70 * 130,)),
                be.reshape(be.transpose(be.from_numpy(b), 0, 1), (512, 256, 1)),
                be.reshape(be.transpose(be.from_numpy(c), 0, 1), (513 * 257,)),
                be.reshape(be.transpose(be.from_numpy(d), 1, 2), (4, 64, 6 * 128)),
                be.reshape(be.transpose(be.from_numpy(e), 0, 2), (96 * 200 * 3,)),
                be.reshape(be.transpose(be.slice(be.from_numpy(g), 1, 3, 192), 0, 1), (192 * 128,)),
                be.concat(be.transpose(be.from_numpy(a), 0, 1), be.transpose(be.from_numpy(a), 0, 1), 0)]
        return N(be, *outs)

    def expect():
        return [a.T.reshape(-1), b.T.reshape(512, 256, 1), c.T.reshape(-1), d.transpose(0, 2, 1, 3).reshape(4, 64, 768),
                e.transpose(2, 1, 0).reshape(-1), g[:, 3:195].T.reshape(-1), np.concatenate([a.T, a.T], 0)]

    return run, expect


_COLS_IN = [f32(610, (1000, 300)), f32(611, (8192, 64)), f32(612, (64, 4096)), f32(613, (70000, 16)), f32(614, (3, 500, 130))]


@case("reduce_over_strided_axis_sum", "red",
      (lambda: [np.abs(x.astype(np.float64)).sum(-2)[..., None] if x.ndim == 2 else np.abs(x.astype(np.float64)).sum(1)[..., None]
                for x in _COLS_IN]))
def _():
    """`sum` over the last axis of transposed views: the reduced axis has a stride, the outputs are contiguous."""
    def run(be):
        return N(be, *[be.sum(be.transpose(be.from_numpy(x), x.ndim - 2, x.ndim - 1)) for x in _COLS_IN])

    return run, (lambda: [x.astype(np.float64).sum(-2)[..., None] for x in _COLS_IN])


@case("reduce_over_strided_axis_max_argmax_u32")
def _():
    xs = [x.copy() for x in _COLS_IN]
    xs[0][::7] = np.float32(9.5)            # equal maxima down a column: the last one wins
    xs[1][5, :] = np.float32(np.nan)
    xs[3][69999, 3] = np.float32(np.inf)
    u = u32(615, (300, 130))
    us = u32(616, (2000, 260), hi=50)       # many ties

    def run(be):
        outs = []
        for x in xs:
            t = be.transpose(be.from_numpy(x), x.ndim - 2, x.ndim - 1)
            outs += [be.max(t), be.argmax(t)]
        tu = be.transpose(be.from_numpy(u), 0, 1)
        outs += [be.sum(tu), be.max(tu), be.argmax(be.transpose(be.from_numpy(us), 0, 1))]
        return N(be, *outs)

    def expect():
        outs = []
        for x in xs:
            t = np.swapaxes(x, -1, -2)
            outs += [max_last_f32(t), argmax_last(t)]
        outs += [(u.astype(np.uint64).sum(0) & 0xFFFFFFFF).astype(np.uint32)[:, None], u.max(0)[:, None], argmax_last(us.T)]
        return outs

    return run, expect


# ---- decode-time linear layers: lazy, grouped by their shared left operand ---------------------------------------
def _linear(be, x, w):
    """`nn::linear_b_param` without bias (stdlib/nn/mod.rs:182-204): x [B,S,K] times w [N,K] transposed."""
    B, _, K = x.shape
    N = w.shape[0]
    return be.matmul(x, be.broadcast(be.transpose(w, 0, 1), (B, K, N)))


for _B, _K, _Ns in ((4, 512, (512, 128, 128)), (1, 1024, (64, 2048)), (8, 388, (300, 8200)), (4, 512, (8192, 8200)),
                    (2, 2304, (8192, 8192, 96, 100, 104)), (4, 2048, (2048, 512, 516)), (3, 4096, (300, 2052)), (2, 2048, (2500,)),
                    (1, 1024, (2048, 1024, 1024)), (4, 3072, (300, 2052))):
    @case(f"linear_group_B{_B}_K{_K}_N{'_'.join(map(str, _Ns))}", "red",
          (lambda B=_B, K=_K, Ns=_Ns: [np.abs(f32(500 + K, (B, 1, K)).astype(np.float64)) @
                                         np.abs(f32(501 + K + i, (n, K)).astype(np.float64)).T
                                         for i, n in enumerate(Ns)]))
    def _(B=_B, K=_K, Ns=_Ns):
        x = f32(500 + K, (B, 1, K))
        ws = [f32(501 + K + i, (n, K)) for i, n in enumerate(Ns)]

        def run(be):
            tx = be.from_numpy(x)
            ys = [_linear(be, tx, be.from_numpy(w)) for w in ws]     # all issued before any is read
            return N(be, *reversed(ys))[::-1]                          # ... and read last one first

        return run, (lambda: [x.astype(np.float64) @ w.astype(np.float64).T for w in ws])


@case("linear_lazy_consumers", "red")
def _():
    """Lazy products consumed through views, element-wise programs, concat and reductions, and one that
    is never read."""
    x = np.abs(f32(520, (4, 1, 640)))      # positive data: no cancellation, so 1e-3 of the value itself applies
    w1, w2, w3 = np.abs(f32(521, (256, 640))), np.abs(f32(522, (256, 640))), np.abs(f32(523, (64, 640)))

    def run(be):
        tx = be.from_numpy(x)
        a, b_, c = (_linear(be, tx, be.from_numpy(w)) for w in (w1, w2, w3))
        _unused = _linear(be, tx, be.from_numpy(w3))
        heads = be.transpose(be.reshape(a, (4, 1, 4, 64)), 1, 2)          # view of a lazy product
        gated = be.mul(a, b_)                                             # two lazy leaves in one program
        cat = be.concat(be.neg(be.slice(c, 2, 32, 32)), be.slice(c, 2, 0, 32), 2)
        tot = be.sum(b_)
        return N(be, heads, gated, cat, tot, c)

    def expect():
        X = x.astype(np.float64)
        A_, B_, C_ = (X @ w.astype(np.float64).T for w in (w1, w2, w3))
        return [A_.reshape(4, 1, 4, 64).transpose(0, 2, 1, 3), A_ * B_, np.concatenate([-C_[..., 32:], C_[..., :32]], -1),
                B_.sum(-1, keepdims=True), C_]

    return run, expect


# ---- SiLU-gated pair of decode-time linear layers (gate / up of an MLP block) ---------------------------------------
for _B, _K, _N in ((4, 512, 4096), (1, 2048, 8192), (3, 388, 4100), (8, 512, 4096), (4, 512, 512), (1, 1024, 4096), (4, 3072, 4100)):
    @case(f"linear_gated_B{_B}_K{_K}_N{_N}", "red")
    def _(B=_B, K=_K, Nn=_N):
        """`silu(x.Wg) * (x.Wu)` as the MLP of the decoder graphs issues it (llama.rs:262-283 with
        nn::silu = x * sigmoid(x), stdlib/nn/mod.rs:130-166).  Rows of one sign: no cancellation inside a
        product, so 1e-3 of the value applies; gate rows alternate in sign to cover both sigmoid tails."""
        x = np.abs(f32(540 + Nn, (B, 1, K)))
        wg = np.abs(f32(541 + Nn, (Nn, K))) * np.float32(8.0 / K)
        wg[::2] *= -1
        wu = np.abs(f32(542 + Nn, (Nn, K))) * np.float32(8.0 / K)

        def run(be):
            tx = be.from_numpy(x)
            g, u = _linear(be, tx, be.from_numpy(wg)), _linear(be, tx, be.from_numpy(wu))
            del tx
            sh = (B, 1, Nn)
            e = be.exp(be.neg(g).move())
            sg = be.div(_const(be, 1.0, sh).move(), be.add(_const(be, 1.0, sh).move(), e.move()).move())
            return N(be, be.mul(be.mul(g.move(), sg.move()).move(), u.move()))

        def expect():
            X = x.astype(np.float64)
            G, U = X @ wg.astype(np.float64).T, X @ wu.astype(np.float64).T
            return [G / (1.0 + np.exp(-G)) * U]

        return run, expect


# ---- residual adds around a decode-time linear layer (the o / down projection of a decoder layer) -------------------
for _B, _K, _N in ((4, 512, 2048), (8, 260, 2052), (1, 1024, 4096), (4, 512, 512), (4, 512, 256), (4, 2048, 2048), (3, 4096, 2052), (2, 2048, 4100), (1, 3072, 2048), (4, 1024, 2052)):
    @case(f"linear_residual_B{_B}_K{_K}_N{_N}", "red")
    def _(B=_B, K=_K, Nn=_N):
        """Sums of three dense terms and a lazy product in the two association orders and every operand
        position the layer loop of the decoder graphs produces (llama.rs:347-365: x + attn, then + mlp)."""
        x = np.abs(f32(560 + Nn, (B, 1, K)))
        w = np.abs(f32(561 + Nn, (Nn, K)))
        ts = [np.abs(f32(562 + Nn + i, (B, 1, Nn))) for i in range(3)]

        def run(be):
            outs = []
            for order in (0, 1):
                for slot in range(4):
                    tx = be.from_numpy(x)
                    t = [be.from_numpy(a) for a in ts]
                    t.insert(slot, _linear(be, tx, be.from_numpy(w)))
                    del tx
                    inner = be.add(t[1].move(), t[2].move())
                    if order == 0:
                        r = be.add(be.add(t[0].move(), inner.move()).move(), t[3].move())
                    else:
                        r = be.add(t[0].move(), be.add(inner.move(), t[3].move()).move())
                    outs.append(r)
            return N(be, *outs)

        def expect():
            P = x.astype(np.float64) @ w.astype(np.float64).T
            return [P + sum(a.astype(np.float64) for a in ts)] * 8

        return run, expect


# ---- products with a fused store whose destination is a part of a larger buffer --------------------------------------
for _axis, _B, _K, _N in ((0, 2, 512, 2048), (1, 1, 1024, 2048), (0, 4, 2048, 2048), (1, 1, 512, 4096)):
    @case(f"linear_fused_store_into_concat_dim{_axis}_B{_B}_K{_K}_N{_N}", "red",
          (lambda: [None] * 6 + [np.float64(8.0)] * 2))   # positive data: 1e-3 of the value; the normed products: of 8
    def _(axis=_axis, B=_B, K=_K, Nn=_N):
        """`concat(prev, h + x.W)`, `concat(prev, t0 + (t1 + t2) + x.W)` and `concat(prev, silu(x.Wg) * x.Wu)` along the
        outermost axis: the open product is computed straight into the second part of the result (a view with an
        offset), both into a fresh buffer and appended in place to a stack this call holds alone; then an RMS norm over
        rows of the stack feeds further products (row sums kept for a part must not be taken for the whole)."""
        r_ = np.random.default_rng(580 + axis + Nn)
        x = np.abs(r_.standard_normal((B, 1, K))).astype(np.float32)
        w, wg, wu = (np.abs(r_.standard_normal((Nn, K))).astype(np.float32) for _ in range(3))
        wg *= np.float32(8.0 / K)
        wu *= np.float32(8.0 / K)
        wg[::2] *= -1
        ts = [np.abs(r_.standard_normal((B, 1, Nn))).astype(np.float32) for _ in range(3)]
        pshape = (3, 1, Nn) if axis == 0 else (1, 3, Nn)
        prev = np.abs(r_.standard_normal(pshape)).astype(np.float32)
        gm = (1.0 + 0.1 * r_.standard_normal(Nn)).astype(np.float32)
        w2 = r_.standard_normal((64, Nn)).astype(np.float32) * np.float32(1.0 / np.sqrt(Nn))

        def run(be):
            def two():
                return be.add(be.from_numpy(ts[0]).move(), _linear(be, be.from_numpy(x), be.from_numpy(w)).move())

            def four():
                inner = be.add(be.from_numpy(ts[1]).move(), be.from_numpy(ts[2]).move())
                return be.add(be.add(be.from_numpy(ts[0]).move(), inner.move()).move(),
                              _linear(be, be.from_numpy(x), be.from_numpy(w)).move())

            def gated():
                tx = be.from_numpy(x)
                g, u = _linear(be, tx, be.from_numpy(wg)), _linear(be, tx, be.from_numpy(wu))
                del tx
                sh = (B, 1, Nn)
                e = be.exp(be.neg(g).move())
                sg = be.div(_const(be, 1.0, sh).move(), be.add(_const(be, 1.0, sh).move(), e.move()).move())
                return be.mul(be.mul(g.move(), sg.move()).move(), u.move())

            outs = []
            for make in (two, four, gated):
                # into the second part of a fresh result
                outs.append(be.concat(be.from_numpy(prev), make().move(), axis))
                # appended in place: the stack is held by this call alone and has room behind it
                stack = be.concat(be.from_numpy(prev[:1] if axis == 0 else prev[:, :1]),
                                  be.from_numpy(prev[1:] if axis == 0 else prev[:, 1:]), axis)
                outs.append(be.concat(stack.move(), make().move(), axis))
            # an RMS norm over the rows of a stack whose last rows came from a fused store, then a product
            for cat in (outs[0], outs[1]):
                rows = int(np.prod(pshape[:2])) + B
                h = be.reshape(cat, (1, rows, Nn)) if rows <= 4 else be.slice(be.reshape(cat, (1, rows, Nn)), 1, rows - 4, 4)
                shp = (1, min(rows, 4), Nn)
                n1 = _rmsnorm_ops(be, h, be.from_numpy(gm), Nn, shp)
                outs.append(_linear(be, n1, be.from_numpy(w2)))
            return N(be, *outs)

        def expect():
            f8 = np.float64
            X = x.astype(f8)
            P = X @ w.astype(f8).T
            G, U = X @ wg.astype(f8).T, X @ wu.astype(f8).T
            vals = [ts[0].astype(f8) + P, sum(t.astype(f8) for t in ts) + P, G / (1.0 + np.exp(-G)) * U]
            if axis == 1:
                vals = [v.reshape(1, B, Nn) for v in vals]
            cats = []
            for v in vals:
                c = np.concatenate([prev.astype(f8), v], axis)
                cats += [c, c]
            outs = list(cats)
            for c in cats[:2]:
                h = c.reshape(1, -1, Nn)[:, -4:]
                n1 = h / np.sqrt((h * h).mean(-1, keepdims=True) + f8(np.float32(1e-5))) * gm.astype(f8)
                outs.append(n1 @ w2.astype(f8).T)
            return outs

        return run, expect


# ---- decode-time attention: q.K^T -> causal soft-max -> p.V as the model graphs issue it ------------------------
def decode_attention_ops(be, q, k_cache, v_cache, rep):
    """One decode step's attention of `LlamaModel` (catgrad-llm-models/src/models/llama.rs:285-345) on a
    cache of T positions: repeat_kv, scores, 1/sqrt(hd), causal mask row T-1 (helpers/tensors.rs:207-224),
    soft-max (stdlib/nn/mod.rs:168-179), context.  q [B, kvH*rep, 1, hd]; caches [B, kvH, T, hd]."""
    B, kvh, T, hd = k_cache.shape
    H = kvh * rep
    S = q.shape[2]          # 1: a decode step; more: a prefill chunk whose last position is T - 1

    def repeat_kv(t):
        t = be.reshape(t.move(), (B, kvh, 1, T, hd))
        t = be.broadcast(t.move(), (B, kvh, rep, T, hd))
        return be.reshape(t.move(), (B, H, T, hd))

    k, v = repeat_kv(k_cache), repeat_kv(v_cache)
    attn = be.matmul(q.move(), be.transpose(k.move(), 2, 3).move())
    sh = (B, H, S, T)
    attn = be.div(attn.move(), _const(be, float(np.sqrt(np.float32(hd))), sh).move())
    ci = be.broadcast(be.arange(T).move(), (T, T))
    cj = be.broadcast(be.reshape(be.arange(T).move(), (T, 1)).move(), (T, T))
    mask = be.cast(be.lt(cj.move(), ci.move()).move(), A.F32)
    mask = be.mul(mask.move(), _const(be, float(F32_MIN), (T, T)).move())
    mask = be.slice(mask.move(), 0, T - S, S)
    attn = be.add(attn.move(), be.broadcast(mask.move(), sh).move())
    m = be.max(attn)
    x = be.sub(attn.move(), be.broadcast(m.move(), sh).move())
    ex = be.exp(x.move())
    ssum = be.sum(ex)
    p = be.div(ex.move(), be.broadcast(ssum.move(), sh).move())
    return be.matmul(p.move(), v.move())


def _np_decode_attention(q, k, v, rep):
    B, kvh, T, hd = k.shape
    S = q.shape[2]
    kk = np.repeat(k.astype(np.float64), rep, axis=1)
    vv = np.repeat(v.astype(np.float64), rep, axis=1)
    s = q.astype(np.float64) @ kk.transpose(0, 1, 3, 2) / np.float64(np.sqrt(np.float32(hd)))
    visible = np.arange(T)[None, :] <= (T - S + np.arange(S))[:, None]      # query at position T - S + i sees keys 0 .. T - S + i
    s = np.where(visible, s, -np.inf)
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    return (e / e.sum(-1, keepdims=True)) @ vv


for _B, _kvh, _rep, _T, _hd in ((2, 2, 4, 300, 64), (1, 3, 1, 1, 64), (2, 1, 8, 63, 64), (1, 2, 2, 65, 128),
                                (4, 8, 4, 1000, 64), (1, 1, 3, 257, 128), (2, 2, 4, 40, 32),
                                # one workgroup per query row in several trips, with and without the split of head_dim, a
                                # batch that does not fill the last eight block indices, caches it takes in two segments and one
                                # beyond its reach
                                (4, 8, 4, 2100, 64), (1, 2, 2, 3000, 128), (5, 8, 4, 700, 64), (9, 1, 8, 1100, 128),
                                (1, 2, 4, 4500, 64), (2, 2, 4, 9000, 64), (1, 1, 2, 5000, 128), (1, 2, 4, 7000, 64),
                                # few query rows at one sequence (the single-sequence decoder shapes)
                                (1, 8, 2, 1100, 128), (1, 3, 3, 640, 64), (2, 4, 4, 2049, 64), (1, 2, 4, 513, 64),
                                # a workgroup per KV head and segment of the cache with five to eight query rows per KV head: in one
                                # trip and in several, both head sizes; a last segment of one position; the longest cache it takes
                                (3, 2, 8, 700, 64), (1, 1, 8, 3000, 64), (1, 1, 8, 2500, 128), (2, 2, 5, 1281, 64), (1, 1, 2, 16384, 64),
                                (1, 1, 4, 16500, 64)):
    @case(f"decode_attention_B{_B}_kv{_kvh}_rep{_rep}_T{_T}_hd{_hd}", "ew_abs")
    def _(B=_B, kvh=_kvh, rep=_rep, T=_T, hd=_hd):
        q = f32(400 + T, (B, kvh * rep, 1, hd))
        k = f32(401 + T, (B, kvh, T, hd))
        v = f32(402 + T, (B, kvh, T, hd))

        def run(be):
            return N(be, decode_attention_ops(be, be.from_numpy(q), be.from_numpy(k), be.from_numpy(v), rep))

        return run, (lambda: [_np_decode_attention(q, k, v, rep)])


# ---- a decode step's attention block: q / k / v projections, rotary embedding, cache append, attention ------------------
def _np_rope(x, cos, sin):
    h = x.shape[-1] // 2
    return cos * x + sin * np.concatenate([-x[..., h:], x[..., :h]], -1)


for _B, _K, _kvh, _rep, _T, _hd, _normed in ((4, 2048, 8, 4, 300, 64, True), (1, 1024, 2, 2, 256, 128, False), (2, 2048, 4, 1, 131, 64, True),
                                              (3, 512, 4, 2, 200, 64, False), (3, 256, 4, 2, 200, 64, False), (4, 2048, 2, 4, 512, 32, False),
                                              # hidden sizes that are no multiple of 1024: a ragged chunk of k in the fused store
                                              (1, 576, 3, 3, 200, 64, True), (4, 576, 3, 3, 300, 64, False), (2, 1536, 4, 2, 131, 64, True),
                                              (3, 2560, 2, 4, 260, 128, True),
                                              # q and k with an RMS norm per head ahead of the embedding (the Qwen3 attention block):
                                              # shapes whose products leave the norm to the launch behind their store (any hidden
                                              # size above 256; head sizes that are no powers of two), and one that does not
                                              (1, 1024, 8, 2, 300, 128, "qk_normed"), (4, 1024, 2, 2, 200, 64, "qk"), (2, 576, 3, 3, 131, 64, "qk_normed"),
                                              (3, 512, 2, 1, 257, 32, "qk"), (1, 2048, 2, 2, 100, 128, "qk_normed"), (2, 256, 2, 2, 90, 64, "qk"),
                                              (4, 2560, 4, 2, 77, 96, "qk_normed"), (2, 1280, 2, 3, 63, 80, "qk"), (3, 4096, 1, 4, 40, 48, "qk_normed")):
    @case(f"decode_qkv_rope_append_B{_B}_K{_K}_kv{_kvh}_rep{_rep}_T{_T}_hd{_hd}{('_' + _normed) if isinstance(_normed, str) else '_normed' if _normed else ''}", "red",
          (lambda n=2 * 3: [np.float64(4.0)] * n))   # projections of order one, rows of the caches likewise: 1e-3 of 4
    def _(B=_B, K=_K, kvh=_kvh, rep=_rep, T=_T, hd=_hd, normed=_normed):
        """Two decode steps of an attention block (llama.rs:285-345): the q / k / v projections of one activation row
        per batch entry (with `normed` the RMS norm of a residual stream that an o projection's store produced),
        heads split off, rotary embedding at the new position (helpers/rope.rs:423-447), k and v appended to caches of
        T rows (helpers/cache.rs:64-74; the first append moves the cache into a buffer with room, the second lands
        behind it), attention over the grown caches.  Where the extents allow it the embedding and the append run in
        the stores of the three products."""
        H = kvh * rep
        qk = isinstance(normed, str)            # an RMS norm over head_dim on q and k (qwen3.rs:249-279)
        normed = normed in (True, "qk_normed")
        r_ = np.random.default_rng(4400 + K + T)
        sc = np.float32(1.0 / np.sqrt(K))
        xs = [r_.standard_normal((B, 1, K)).astype(np.float32) for _ in range(2)]
        res = [r_.standard_normal((B, 1, K)).astype(np.float32) for _ in range(2)]
        wo = r_.standard_normal((K, K)).astype(np.float32) * sc
        gm = (1.0 + 0.1 * r_.standard_normal(K)).astype(np.float32)
        wq = r_.standard_normal((H * hd, K)).astype(np.float32) * sc
        wk = r_.standard_normal((kvh * hd, K)).astype(np.float32) * sc
        wv = r_.standard_normal((kvh * hd, K)).astype(np.float32) * sc
        ck = r_.standard_normal((B, kvh, T, hd)).astype(np.float32)
        cv = r_.standard_normal((B, kvh, T, hd)).astype(np.float32)
        ang = r_.uniform(0, 6.28, (T + 2, hd)).astype(np.float32)
        cos_t, sin_t = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        gq = (1.0 + 0.1 * r_.standard_normal(hd)).astype(np.float32)
        gk = (1.0 + 0.1 * r_.standard_normal(hd)).astype(np.float32)

        def run(be):
            k_cache, v_cache = be.from_numpy(ck), be.from_numpy(cv)
            tcos, tsin = be.from_numpy(cos_t), be.from_numpy(sin_t)
            weights = [be.from_numpy(w) for w in (wq, wk, wv)]
            outs = []
            for step in range(2):
                pos = T + step
                if normed:
                    h = be.add(be.from_numpy(res[step]).move(), _linear(be, be.from_numpy(xs[step]), be.from_numpy(wo)).move())
                    xn = _rmsnorm_ops(be, h, be.from_numpy(gm), K, (B, 1, K))
                    del h
                else:
                    xn = be.from_numpy(xs[step])
                q, k, v = (_linear(be, xn, w) for w in weights)
                del xn

                def heads(t, n):
                    return be.transpose(be.reshape(t.move(), (B, 1, n, hd)).move(), 1, 2)

                def rope(t, n):
                    sh = (B, n, 1, hd)
                    c = be.broadcast(be.reshape(be.slice(tcos, 0, pos, 1).move(), (1, 1, 1, hd)).move(), sh)
                    s_ = be.broadcast(be.reshape(be.slice(tsin, 0, pos, 1).move(), (1, 1, 1, hd)).move(), sh)
                    rot = _rot_half(be, t, hd // 2)
                    return be.add(be.mul(c.move(), t.move()).move(), be.mul(s_.move(), rot.move()).move())

                q, k, v = heads(q, H), heads(k, kvh), heads(v, kvh)
                if qk:
                    def head_norm(t, n, g):
                        flat = be.reshape(t.move(), (B * n, hd))
                        normed_t = _rmsnorm_ops(be, flat, be.from_numpy(g), hd, (B * n, hd))
                        del flat   # (the graph interpreter gives every handle away at its last use)
                        return be.reshape(normed_t.move(), (B, n, 1, hd))

                    q, k = head_norm(q, H, gq), head_norm(k, kvh, gk)
                q, k = rope(q, H), rope(k, kvh)
                k_cache = be.concat(k_cache.move(), k.move(), 2)
                v_cache = be.concat(v_cache.move(), v.move(), 2)
                outs.append(decode_attention_ops(be, q, k_cache.clone(), v_cache.clone(), rep))
                outs += [be.slice(k_cache, 2, pos, 1), be.slice(v_cache, 2, pos, 1)]
            return N(be, *outs)

        def expect():
            f8 = np.float64
            K_, V_ = ck.astype(f8), cv.astype(f8)
            outs = []
            for step in range(2):
                pos = T + step
                x = xs[step].astype(f8)
                if normed:
                    h = res[step].astype(f8) + x @ wo.astype(f8).T
                    x = h / np.sqrt((h * h).mean(-1, keepdims=True) + 1e-5) * gm.astype(f8)
                q = (x @ wq.astype(f8).T).reshape(B, 1, H, hd).transpose(0, 2, 1, 3)
                k = (x @ wk.astype(f8).T).reshape(B, 1, kvh, hd).transpose(0, 2, 1, 3)
                v = (x @ wv.astype(f8).T).reshape(B, 1, kvh, hd).transpose(0, 2, 1, 3)
                if qk:
                    q = q / np.sqrt((q * q).mean(-1, keepdims=True) + 1e-5) * gq.astype(f8)
                    k = k / np.sqrt((k * k).mean(-1, keepdims=True) + 1e-5) * gk.astype(f8)
                c, s_ = cos_t[pos].astype(f8), sin_t[pos].astype(f8)
                q, k = _np_rope(q, c, s_), _np_rope(k, c, s_)
                K_, V_ = np.concatenate([K_, k], 2), np.concatenate([V_, v], 2)
                outs += [_np_decode_attention(q, K_, V_, rep), k, v]
            return outs

        return run, expect


# ---- prefill attention: many query positions per head, causal ---------------------------------------------------------
for _B, _kvh, _rep, _S, _T, _hd in ((1, 2, 4, 48, 48, 64), (2, 1, 1, 128, 128, 64), (1, 2, 2, 200, 333, 64), (2, 2, 4, 96, 96, 64),
                                     (1, 1, 3, 70, 70, 64), (1, 1, 1, 9, 500, 64), (1, 2, 2, 64, 64, 128), (2, 1, 4, 200, 333, 128),
                                     (1, 2, 2, 40, 40, 32),
                                     # few workgroups: the keys of a row tile cut over several of them and merged (parts without a
                                     # visible key for some rows, a last part of one tile, both head sizes, a prompt behind a cache)
                                     (1, 2, 2, 1024, 1024, 128), (1, 3, 3, 512, 512, 64), (1, 1, 4, 300, 1500, 64), (2, 1, 2, 130, 777, 128)):
    @case(f"prefill_attention_B{_B}_kv{_kvh}_rep{_rep}_S{_S}_T{_T}_hd{_hd}", "ew_abs")
    def _(B=_B, kvh=_kvh, rep=_rep, S=_S, T=_T, hd=_hd):
        """q [B, H, S, hd] against caches of T >= S positions (the last S of them are the queries' own): row tiles
        that end inside a head or span two heads, a cache longer than the chunk, key tiles cut by the diagonal,
        head sizes the one-pass kernel declines."""
        q = f32(450 + S + T, (B, kvh * rep, S, hd))
        k = f32(451 + S + T, (B, kvh, T, hd))
        v = f32(452 + S + T, (B, kvh, T, hd))

        def run(be):
            return N(be, decode_attention_ops(be, be.from_numpy(q), be.from_numpy(k), be.from_numpy(v), rep))

        return run, (lambda: [_np_decode_attention(q, k, v, rep)])


# ---- deferred row programs: sum / max that stay inside a fused expression -----------------------------
def _const(be, v, shape, dt=np.float32):
    return be.broadcast(be.from_numpy(np.array(v, dt)), shape)


def _np_softmax(x):
    x = x.astype(np.float64)
    e = np.exp(x - x.max(-1, keepdims=True))
    return e / e.sum(-1, keepdims=True)


for _shape in ((1, 5), (3, 7, 33), (4, 8, 1, 260), (2, 3000), (5, 1), (130, 4), (2, 3, 2052)):
    @case(f"rows_softmax_{'x'.join(map(str, _shape))}", "ew")
    def _(shape=_shape):
        a = f32(200 + len(shape) + shape[-1], shape, 2.0)
        return (lambda be: N(be, softmax_ops(be, be.from_numpy(a)))), (lambda: [_np_softmax(a)])


@case("rows_attention_softmax_scale_mask", "ew")
def _():
    """softmax(scores * scale + mask) with the mask broadcast over batch and heads, scores a strided view."""
    B, H, S, T = 2, 3, 5, 64
    sc = f32(210, (B, S, H, T), 1.5)
    mask = np.where(np.arange(T)[None, :] <= np.arange(S)[:, None] + (T - S), 0.0, F32_MIN).astype(np.float32)

    def run(be):
        x = be.transpose(be.from_numpy(sc), 1, 2)  # [B,H,S,T] view
        shp = (B, H, S, T)
        x = be.mul(x, _const(be, 0.125, shp))
        x = be.add(x, be.broadcast(be.from_numpy(mask.reshape(1, 1, S, T)), shp))
        return N(be, softmax_ops(be, x))

    return run, (lambda: [_np_softmax(sc.transpose(0, 2, 1, 3).astype(np.float64) * 0.125 + mask)])


for _n in (64, 576, 2048):
    @case(f"rows_rmsnorm_{_n}", "ew")
    def _(n=_n):
        x = f32(220 + n, (3, 2, n), 1.7)
        r = f32(221 + n, (3, 2, n), 0.3)
        g = f32(222 + n, (n,), 1.0)

        def run(be):
            shp = (3, 2, n)
            h = be.add(be.from_numpy(x), be.from_numpy(r))  # residual add feeding the norm
            s = be.sum(be.mul(h, h))
            mean = be.div(s, _const(be, float(n), (3, 2, 1)))
            rms = be.pow(be.add(mean, _const(be, 1e-5, (3, 2, 1))), _const(be, 0.5, (3, 2, 1)))
            y = be.div(h, be.broadcast(rms, shp))
            return N(be, be.mul(y, be.broadcast(be.from_numpy(g), shp)), h)

        def expect():
            h = (x + r).astype(np.float64)
            y = h / np.sqrt((h * h).mean(-1, keepdims=True) + np.float64(np.float32(1e-5)))
            return [y * g, x + r]

        return run, expect


def _rmsnorm_ops(be, h, gamma, n, shp):
    """`rmsnorm` of the decoder graphs (stdlib/nn/mod.rs:208-232): x / sqrt(mean(x^2) + eps) * gamma."""
    one = shp[:-1] + (1,)
    # every intermediate handle is given away at its last use, as the graph interpreter does
    s = be.sum(be.mul(h, h).move())
    mean = be.div(s.move(), _const(be, float(n), one).move())
    rms = be.pow(be.add(mean.move(), _const(be, 1e-5, one).move()).move(), _const(be, 0.5, one).move())
    return be.mul(be.div(h, be.broadcast(rms.move(), shp).move()).move(), be.broadcast(gamma.move(), shp).move())


for _B, _H, _F, _read_norms in ((4, 2048, 4096, False), (2, 2048, 4096, True), (3, 4096, 8192, False), (4, 512, 4096, False), (4, 256, 4096, False), (1, 2048, 4096, False),
                                 (1, 1024, 3072, False), (4, 3072, 4096, False),
                                 # hidden and MLP sizes that are no multiples of 1024 (ragged chunks of k, few columns)
                                 (1, 576, 1536, False), (4, 576, 1536, True), (2, 1536, 2560, False), (3, 2560, 6912, False)):
    @case(f"decoder_block_B{_B}_H{_H}_F{_F}{'_norms_read' if _read_norms else ''}", "red",
          (lambda n=5 + 2 * _read_norms: [np.float64(4.0)] * n))   # every output is of order one: 1e-3 of 4
    def _(B=_B, H=_H, F=_F, read_norms=_read_norms):
        """The dense part of a decoder layer at decode time (llama.rs:347-365): residual add of the o projection,
        RMS norm, gate / up / SiLU, down projection, residual add, RMS norm, q / k / v projections.  Where the
        extents allow it the residual adds run in the stores of the o / down products and the norms in the loads of
        the products behind them; with `norms_read` the norms are also read back, which makes them run on their own."""
        rng_ = np.random.default_rng(700 + B + H)
        sc = np.float32(1.0 / np.sqrt(H))
        x0 = rng_.standard_normal((B, 1, H)).astype(np.float32)
        a0 = rng_.standard_normal((B, 1, H)).astype(np.float32)
        wo = rng_.standard_normal((H, H)).astype(np.float32) * sc
        wg = rng_.standard_normal((F, H)).astype(np.float32) * sc
        wu = rng_.standard_normal((F, H)).astype(np.float32) * sc
        wd = rng_.standard_normal((H, F)).astype(np.float32) * np.float32(1.0 / np.sqrt(F))
        wq = rng_.standard_normal((H, H)).astype(np.float32) * sc
        wk = rng_.standard_normal((H // 4, H)).astype(np.float32) * sc
        wv = rng_.standard_normal((H // 4, H)).astype(np.float32) * sc
        g1 = (1.0 + 0.1 * rng_.standard_normal(H)).astype(np.float32)
        g2 = (1.0 + 0.1 * rng_.standard_normal(H)).astype(np.float32)

        def run(be):
            shp, fs = (B, 1, H), (B, 1, F)
            h1 = be.add(be.from_numpy(x0).move(), _linear(be, be.from_numpy(a0), be.from_numpy(wo)).move())
            n1 = _rmsnorm_ops(be, h1, be.from_numpy(g1), H, shp)
            g, u = _linear(be, n1, be.from_numpy(wg)), _linear(be, n1, be.from_numpy(wu))
            e = be.exp(be.neg(g).move())
            sg = be.div(_const(be, 1.0, fs).move(), be.add(_const(be, 1.0, fs).move(), e.move()).move())
            act = be.mul(be.mul(g.move(), sg.move()).move(), u.move())
            h2 = be.add(h1, _linear(be, act, be.from_numpy(wd)).move())
            del act
            n2 = _rmsnorm_ops(be, h2, be.from_numpy(g2), H, shp)
            q, k, v = (_linear(be, n2, be.from_numpy(w)) for w in (wq, wk, wv))
            outs = [q, k, v, h2, h1]
            if read_norms:
                outs += [n1, n2]
            else:
                del n1, n2
            return N(be, *outs)

        def expect():
            f8 = np.float64

            def norm(h, gm):
                return h / np.sqrt((h * h).mean(-1, keepdims=True) + f8(np.float32(1e-5))) * gm.astype(f8)

            h1 = x0.astype(f8) + a0.astype(f8) @ wo.astype(f8).T
            n1 = norm(h1, g1)
            G, U = n1 @ wg.astype(f8).T, n1 @ wu.astype(f8).T
            act = G / (1.0 + np.exp(-G)) * U
            h2 = h1 + act @ wd.astype(f8).T
            n2 = norm(h2, g2)
            outs = [n2 @ wq.astype(f8).T, n2 @ wk.astype(f8).T, n2 @ wv.astype(f8).T, h2, h1]
            return outs + ([n1, n2] if read_norms else [])

        return run, expect


@case("rows_reduced_results_alone", "red")
def _():
    """Row results that are read back without being broadcast: a lone reduce, ops then reduce,
    reduce then ops, and ops on two row results."""
    a = np.abs(f32(230, (6, 5, 130), 1.0)) + np.float32(0.5)
    b = np.abs(f32(231, (6, 5, 130), 1.0)) + np.float32(0.5)
    w = f32(232, (6, 5, 1), 1.0)

    def run(be):
        ta, tb, tw = be.from_numpy(a), be.from_numpy(b), be.from_numpy(w)
        s1 = be.sum(ta)
        s2 = be.sum(be.mul(ta, tb))
        s3 = be.add(be.div(be.sum(ta), _const(be, 130.0, (6, 5, 1))), tw)
        s4 = be.div(be.sum(be.mul(ta, tb)), be.max(tb))
        s5 = be.mul(be.max(ta), be.exp(be.neg(be.max(ta))))
        return N(be, s1, s2, s3, s4, s5, be.max(ta))

    def expect():
        A64, B64 = a.astype(np.float64), b.astype(np.float64)
        m = A64.max(-1, keepdims=True)
        return [A64.sum(-1, keepdims=True), (A64 * B64).sum(-1, keepdims=True), A64.mean(-1, keepdims=True) + w,
                (A64 * B64).sum(-1, keepdims=True) / B64.max(-1, keepdims=True), m * np.exp(-m), m]

    return run, expect


@case("rows_u32_wrapping")
def _():
    a = u32(240, (4, 3, 37))

    def run(be):
        t = be.from_numpy(a)
        shp = (4, 3, 37)
        y = be.add(t, be.broadcast(be.sum(t), shp))
        z = be.sub(be.broadcast(be.max(t), shp), t)
        q = be.div(be.broadcast(be.max(t), shp), be.add(t, _const(be, 1, shp, np.uint32)))
        return N(be, y, z, q, be.add(be.sum(t), be.max(t)))

    def expect():
        s = a.astype(np.uint64).sum(-1, keepdims=True).astype(np.uint32)
        m = a.max(-1, keepdims=True)
        d = (a.astype(np.uint64) + 1).astype(np.uint32)
        with np.errstate(divide="ignore"):
            q = np.where(d == 0, 0, m // np.maximum(d, 1)).astype(np.uint32)
        return [a + s, m - a, q, s + m]

    return run, expect


@case("rows_shared_and_viewed_results", "ew")
def _():
    """Row results with several users, and views / concats of row programs (which end the deferral)."""
    a = f32(250, (3, 4, 24), 1.0)
    b = f32(251, (3, 4, 24), 1.0)

    def run(be):
        ta, tb = be.from_numpy(a), be.from_numpy(b)
        shp = (3, 4, 24)
        m = be.max(ta)
        bm = be.broadcast(m, shp)
        o1 = be.sub(ta, bm)
        o2 = be.add(tb, bm)                               # bm used twice
        o3 = be.add(be.transpose(m, 0, 1), _const(be, 1.0, (4, 3, 1)))   # view of a row result
        sm = softmax_ops(be, ta)
        o4 = be.transpose(sm, 1, 2)                       # view of a full row program
        o5 = be.concat(softmax_ops(be, tb), ta, 2)        # row program written into a strided destination
        o6 = be.concat(be.sum(ta), be.max(tb), 2)         # row results as concat operands
        o7 = be.reshape(softmax_ops(be, ta), (12, 24))
        o8 = be.slice(softmax_ops(be, ta), 2, 3, 7)
        o9 = be.broadcast(be.sum(ta), (3, 4, 5))          # row result broadcast to another length
        o10 = be.broadcast(be.sum(ta), (2, 3, 4, 24))     # ... and with a rank increase
        return N(be, o1, o2, o3, o4, o5, o6, o7, o8, o9, o10)

    def expect():
        A64, B64 = a.astype(np.float64), b.astype(np.float64)
        m = A64.max(-1, keepdims=True)
        s = A64.sum(-1, keepdims=True)
        return [A64 - m, B64 + m, m.transpose(1, 0, 2) + 1.0, _np_softmax(a).transpose(0, 2, 1),
                np.concatenate([_np_softmax(b), A64], 2), np.concatenate([s, B64.max(-1, keepdims=True)], 2),
                _np_softmax(a).reshape(12, 24), _np_softmax(a)[:, :, 3:10], np.broadcast_to(s, (3, 4, 5)),
                np.broadcast_to(s, (2, 3, 4, 24))]

    return run, expect
CASES[-1].kind = "ew_abs"


@case("rows_many_reduces_and_mixed_lengths", "ew")
def _():
    """Three reduces in one program, a fourth that does not fit, layer-norm style centring, and row
    results of different row lengths meeting in one op."""
    a = f32(260, (5, 48), 1.0)
    c = np.abs(f32(261, (5, 20), 1.0)) + np.float32(1.0)

    def run(be):
        ta, tc = be.from_numpy(a), be.from_numpy(c)
        shp = (5, 48)
        y = softmax_ops(be, ta)
        z = be.div(y, be.broadcast(be.max(y), shp))             # 3 reduces
        z4 = be.sum(z)                                           # a 4th
        mean = be.div(be.sum(ta), _const(be, 48.0, (5, 1)))
        cen = be.sub(ta, be.broadcast(mean, shp))
        var = be.div(be.sum(be.mul(cen, cen)), _const(be, 48.0, (5, 1)))
        ln = be.div(cen, be.broadcast(be.pow(be.add(var, _const(be, 1e-5, (5, 1))), _const(be, 0.5, (5, 1))), shp))
        mix = be.add(be.sum(tc), be.max(ta))                     # row lengths 20 and 48
        return N(be, z, z4, ln, mix)

    def expect():
        A64 = a.astype(np.float64)
        y = _np_softmax(a)
        z = y / y.max(-1, keepdims=True)
        cen = A64 - A64.mean(-1, keepdims=True)
        ln = cen / np.sqrt((cen * cen).mean(-1, keepdims=True) + np.float64(np.float32(1e-5)))
        return [z, z.sum(-1, keepdims=True), ln, c.astype(np.float64).sum(-1, keepdims=True) + A64.max(-1, keepdims=True)]

    return run, expect
CASES[-1].kind = "ew_abs"


@case("rows_degenerate_extents")
def _():
    a = rng(270).integers(-9, 10, size=(4, 1)).astype(np.float32)
    e = np.zeros((0, 7), np.float32)

    def run(be):
        ta, te = be.from_numpy(a), be.from_numpy(e)
        o1 = be.add(be.broadcast(be.sum(ta), (4, 1)), ta)
        o2 = be.sub(ta, be.broadcast(be.max(ta), (4, 1)))
        o3 = be.broadcast(be.sum(te), (0, 7))
        z = be.zeros((3, 0), A.F32)
        return N(be, o1, o2, o3, be.sum(z), be.max(z), be.add(be.sum(z), be.max(be.zeros((3, 5), A.F32))))

    def expect():
        return [a + a, a - a, e, np.zeros((3, 1), np.float32), np.full((3, 1), F32_MIN), np.zeros((3, 1), np.float32)]

    return run, expect


# ---- mixture-of-experts routing as Qwen3's MoE layer issues it (qwen3.rs:125-194) ------------------------------------
for _S, _E, _k, _H, _I in ((1, 8, 2, 256, 512), (16, 8, 2, 256, 512), (5, 4, 3, 128, 320)):
    @case(f"moe_topk_index_grouped_matmul_S{_S}_E{_E}_k{_k}", "red", (lambda: [np.float64(1.0)]))
    def _(S=_S, E=_E, k=_k, H=_H, I=_I):
        """soft-max router -> `topk` -> per chosen expert `index` on the [E, I, H] stacks -> batched matmul with one
        row per token ([S, 1, H] x [S, H, I]) -> SiLU * up -> down -> weighted sum (norm_topk_prob).  Outputs are of
        order 0.1: 1e-3 of 1 is the bound."""
        for seed in range(640, 740):     # the first seed whose router probabilities leave every top-k choice clear
            r_ = np.random.default_rng(seed + S + E)
            x = r_.standard_normal((1, S, H)).astype(np.float32)
            wr = r_.standard_normal((E, H)).astype(np.float32) * np.float32(4.0 / np.sqrt(H))     # spread router logits
            pr = _np_softmax((x.astype(np.float64) @ wr.astype(np.float64).T)[0])
            srt = np.sort(pr, -1)[:, ::-1]
            if (srt[:, :k] - srt[:, 1:k + 1]).min() > 2e-3:
                break
        wg = r_.standard_normal((E, I, H)).astype(np.float32) * np.float32(1.0 / np.sqrt(H))
        wu = r_.standard_normal((E, I, H)).astype(np.float32) * np.float32(1.0 / np.sqrt(H))
        wd = r_.standard_normal((E, H, I)).astype(np.float32) * np.float32(1.0 / np.sqrt(I))
        assert (srt[:, :k] - srt[:, 1:k + 1]).min() > 2e-3, "router probabilities too close for a stable top-k"

        def run(be):
            tx = be.from_numpy(x)
            routed = softmax_ops(be, _linear(be, tx, be.from_numpy(wr)))
            vals, idxs = be.topk(routed, k)
            sh = (S, k)
            idxs, vals = be.reshape(idxs, sh), be.reshape(vals, sh)
            vals = be.div(vals, be.broadcast(be.sum(vals), sh))
            fullx = be.transpose(tx, 0, 1)                                  # [S, 1, H]
            sumk = _const(be, 0.0, (S, 1, H))
            ga, ua, da = be.from_numpy(wg), be.from_numpy(wu), be.from_numpy(wd)
            for i in range(k):
                idx = be.slice(idxs, 1, i, 1)
                val = be.slice(vals, 1, i, 1)
                g = be.matmul(fullx, be.transpose(be.index(ga, 0, idx), 1, 2))
                u = be.matmul(fullx, be.transpose(be.index(ua, 0, idx), 1, 2))
                one = _const(be, 1.0, (S, 1, I))
                act = be.mul(be.mul(g, be.div(one, be.add(one, be.exp(be.neg(g))))), u)
                y = be.matmul(act, be.transpose(be.index(da, 0, idx), 1, 2))
                v = be.broadcast(be.reshape(val, (S, 1, 1)), (S, 1, H))
                sumk = be.add(sumk, be.mul(y, v))
            return N(be, be.transpose(sumk, 0, 1))

        def expect():
            f8 = np.float64
            out = np.zeros((S, H))
            for t in range(S):
                order = np.argsort(-pr[t], kind="stable")[:k]
                w = pr[t][order] / pr[t][order].sum()
                for e, wt in zip(order, w):
                    g = wg[e].astype(f8) @ x[0, t].astype(f8)
                    u = wu[e].astype(f8) @ x[0, t].astype(f8)
                    out[t] += wt * (wd[e].astype(f8) @ (g / (1.0 + np.exp(-g)) * u))
            return [out[None]]

        return run, expect


def by_name(name):
    for c in CASES:
        if c.name == name:
            return c
    raise KeyError(name)


def assert_close(kind, got, exp, scale=None, name=""):
    """Tolerance of each kind, written out (see module docstring)."""
    got, exp = np.asarray(got), np.asarray(exp)
    assert got.shape == exp.shape, f"{name}: shape {got.shape} != {exp.shape}"
    if kind == "exact":
        if got.dtype == np.float32:
            e32 = exp.astype(np.float32)
            nan_ok = np.isnan(got) & np.isnan(e32)
            same = (got == e32) | nan_ok
            assert same.all(), f"{name}: {np.count_nonzero(~same)} f32 mismatches, first at {np.argwhere(~same)[:3].tolist()}"
        else:
            np.testing.assert_array_equal(got, exp.astype(got.dtype), err_msg=name)
    elif kind == "ew":
        np.testing.assert_allclose(got.astype(np.float64), exp.astype(np.float64), rtol=1e-4, atol=1e-6, err_msg=name)
    elif kind == "ew_abs":  # element-wise math downstream of a row sum: the sum's rounding shows as absolute error
        np.testing.assert_allclose(got.astype(np.float64), exp.astype(np.float64), rtol=1e-4, atol=1e-5, err_msg=name)
    elif kind in ("ulp_f16", "ulp_bf16"):
        # one unit in the last place of the 16-bit dtype: 2^-10 (f16, 11-bit significand) resp. 2^-7 (bf16, 8-bit)
        # of the value at most, plus the spacing of f16 subnormals
        rtol, atol = (2.0 ** -10, 2.0 ** -24) if kind == "ulp_f16" else (2.0 ** -7, 1e-38)
        np.testing.assert_allclose(got.astype(np.float64), exp.astype(np.float64), rtol=rtol, atol=atol, err_msg=name)
    elif kind == "ulp_f8":  # one unit in the last place of E4M3 (4-bit significand), plus the spacing of its subnormals
        np.testing.assert_allclose(got.astype(np.float64), exp.astype(np.float64), rtol=2.0 ** -3, atol=2.0 ** -9, err_msg=name)
    elif kind == "red":
        s = np.asarray(scale, dtype=np.float64) if scale is not None else np.abs(exp.astype(np.float64))
        err = np.abs(got.astype(np.float64) - exp.astype(np.float64))
        bound = 1e-3 * np.maximum(s, 1e-30)
        assert (err <= bound).all(), f"{name}: max err/scale {np.max(err / np.maximum(s, 1e-30)):.3e} > 1e-3"
    else:
        raise ValueError(kind)


import cases_half  # noqa: E402,F401  (appends the 16-bit float cases to CASES)
import cases_fp8  # noqa: E402,F401  (appends the fp8 cases to CASES)

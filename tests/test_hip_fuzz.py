"""Seeded random op graphs, HipBackend against the CPU oracle.

Each graph is a short random program over a few small f32 tensors: element-wise ops, row reductions broadcast
back over their rows, views (transpose / slice / reshape / broadcast), last- and inner-axis concats, casts and a
gather — the mix that exercises the deferred-program engine (splicing, shared sub-expressions, row programs,
piecewise leaves, views of deferred results) in combinations the hand-written cases do not enumerate.  Every
node carries a bound on its magnitude, graphs stay below 1e6, and the comparison is the element-wise tolerance of
the contract (rtol 1e-4) plus an absolute term of 1e-5 of the node's bound, which covers differences that a
subtraction of nearly equal values amplifies."""
import os

import numpy as np
import pytest

from catgrad_amd import _abi as A

pytestmark = pytest.mark.gpu

# CG_FUZZ_SEED_OFFSET=n runs every seeded test below on seeds n, n + 1, ... instead of 0, 1, ... (more of the same fuzz)
SEED0 = int(os.environ.get("CG_FUZZ_SEED_OFFSET", "0"))

LIMIT = 1e6


class Node:
    """`fn(be, *parent tensors)` builds this node; `hi` bounds |values|; `exact` says that every op on the way
    here rounds identically on any IEEE f32 implementation (no exp / sin / cos, no sum whose order may differ), so
    a discontinuous op (floor, round, a comparison, a mask, a truncating cast) may follow it."""

    def __init__(self, fn, parents, shape, hi, exact):
        self.fn, self.parents, self.shape, self.hi, self.exact = fn, parents, tuple(shape), hi, exact


def const(be, v, shape):
    return be.broadcast(be.from_numpy(np.array(v, np.float32)), shape)


def random_graph(rng):
    """Returns (inputs, nodes, outputs): numpy inputs, all nodes in build order, and the nodes to read back."""
    depth = int(rng.integers(6, 30))
    base = (int(rng.integers(1, 4)), int(rng.integers(1, 7)), int(rng.choice([1, 3, 8, 16, 33, 64, 130, 256, 1000, 2048])))
    inputs = [rng.uniform(0.25, 2.0, size=base).astype(np.float32) for _ in range(3)]
    nodes = [Node(None, (), base, 2.0, True) for _ in range(3)]

    def pick(shape=None):
        c = [n for n in nodes if shape is None or n.shape == tuple(shape)]
        return c[int(rng.integers(0, len(c)))]

    def add(fn, parents, shape, hi, inexact=False, needs_exact=()):
        if hi <= LIMIT and all(s > 0 for s in shape) and all(p.exact for p in needs_exact):
            nodes.append(Node(fn, parents, shape, hi, not inexact and all(p.exact for p in parents)))

    kinds = ["unary", "binary", "binary", "binary", "where", "rowsum", "rowmax", "transpose", "slice", "reshape",
             "rotate_half", "concat_last", "concat_inner", "cast", "index", "scalar"]
    for _ in range(depth):
        kind = str(rng.choice(kinds))
        x = pick()
        last = len(x.shape) - 1
        if kind == "unary":
            op = str(rng.choice(["neg", "gauss", "floor", "round", "sin", "cos", "square"]))
            if op == "gauss":      # exp(-x^2), in (0, 1]
                add(lambda be, a: be.exp(be.neg(be.mul(a, a))), (x,), x.shape, 1.0, inexact=True)
            elif op == "square":
                add(lambda be, a: be.mul(a, a), (x,), x.shape, x.hi * x.hi)
            elif op in ("sin", "cos"):
                if x.hi <= 64.0:   # the contract's tolerance for sin / cos holds for moderate arguments
                    add(lambda be, a, op=op: getattr(be, op)(a), (x,), x.shape, 1.0, inexact=True)
            else:
                add(lambda be, a, op=op: getattr(be, op)(a), (x,), x.shape, x.hi + 1.0, needs_exact=() if op == "neg" else (x,))
        elif kind == "binary":
            y = pick(x.shape)
            op = str(rng.choice(["add", "mul", "sub", "ratio", "lt", "gte"]))
            if op == "ratio":      # x / (y^2 + 0.5)
                add(lambda be, a, b, s=x.shape: be.div(a, be.add(be.mul(b, b), const(be, 0.5, s))), (x, y), x.shape, 2 * x.hi)
            else:
                hi = {"add": x.hi + y.hi, "sub": x.hi + y.hi, "mul": x.hi * y.hi}.get(op, 1.0)
                add(lambda be, a, b, op=op: getattr(be, op)(a, b), (x, y), x.shape, hi, needs_exact=(x, y) if op in ("lt", "gte") else ())
        elif kind == "where":
            y, m = pick(x.shape), pick(x.shape)
            add(lambda be, a, b, c, s=x.shape: be.where_cond(be.sub(c, const(be, 1.0, s)), a, b), (x, y, m), x.shape, max(x.hi, y.hi),
                needs_exact=(m,))
        elif kind == "rowsum":     # x / (1 + sum x^2): positive terms, no cancellation inside the sum
            add(lambda be, a, s=x.shape: be.div(a, be.add(be.broadcast(be.sum(be.mul(a, a)), s), const(be, 1.0, s))), (x,), x.shape, x.hi,
                inexact=True)
        elif kind == "rowmax":     # x - max x, the softmax shift
            add(lambda be, a, s=x.shape: be.sub(a, be.broadcast(be.max(a), s)), (x,), x.shape, 2 * x.hi)
        elif kind == "transpose" and len(x.shape) >= 2:
            i, j = sorted(rng.choice(len(x.shape), size=2, replace=False).tolist())
            shp = list(x.shape)
            shp[i], shp[j] = shp[j], shp[i]
            add(lambda be, a, i=i, j=j: be.transpose(a, i, j), (x,), shp, x.hi)
        elif kind == "slice":
            d = int(rng.integers(0, len(x.shape)))
            if x.shape[d] >= 2:
                start = int(rng.integers(0, x.shape[d] - 1))
                ln = int(rng.integers(1, x.shape[d] - start + 1))
                shp = list(x.shape)
                shp[d] = ln
                add(lambda be, a, d=d, start=start, ln=ln: be.slice(a, d, start, ln), (x,), shp, x.hi)
        elif kind == "reshape":
            n = int(np.prod(x.shape))
            shp = (n,) if rng.random() < 0.3 else (n // x.shape[-1], x.shape[-1])
            add(lambda be, a, shp=shp: be.reshape(a, shp), (x,), shp, x.hi)
        elif kind == "rotate_half":    # concat(-x[.., h:], x[.., :h]): one tensor read piecewise
            h = x.shape[-1] // 2
            if h >= 1:
                w = x.shape[-1]
                add(lambda be, a, h=h, w=w, last=last: be.concat(be.neg(be.slice(a, last, h, w - h)), be.slice(a, last, 0, h), last),
                    (x,), x.shape, x.hi)
        elif kind == "concat_last":
            y = pick(x.shape)
            add(lambda be, a, b, last=last: be.concat(a, b, last), (x, y), x.shape[:-1] + (2 * x.shape[-1],), max(x.hi, y.hi))
        elif kind == "concat_inner":
            y = pick(x.shape)
            d = int(rng.integers(0, len(x.shape)))
            shp = list(x.shape)
            shp[d] *= 2
            add(lambda be, a, b, d=d: be.concat(a, b, d), (x, y), shp, max(x.hi, y.hi))
        elif kind == "cast":           # f32 -> u32 -> f32 of a non-negative value: truncation
            add(lambda be, a, s=x.shape: be.cast(be.cast(be.mul(be.mul(a, a), const(be, 7.0, s)), A.U32), A.F32), (x,), x.shape,
                7 * x.hi * x.hi, needs_exact=(x,))
        elif kind == "index":
            d = int(rng.integers(0, len(x.shape)))
            ids = rng.integers(0, x.shape[d], size=int(rng.integers(1, 6))).astype(np.uint32)
            shp = list(x.shape)
            shp[d] = len(ids)
            add(lambda be, a, d=d, ids=ids: be.index(a, d, be.from_numpy(ids)), (x,), shp, x.hi)
        elif kind == "scalar":
            c = float(rng.uniform(0.5, 1.5))
            add(lambda be, a, c=c, s=x.shape: be.mul(a, const(be, c, s)), (x,), x.shape, 1.5 * x.hi)
    cand = np.arange(3, len(nodes))
    outs = [nodes[int(i)] for i in rng.choice(cand, size=min(4, len(cand)), replace=False)] if len(cand) else [nodes[0]]
    return inputs, nodes, outs


def evaluate(be, inputs, nodes, outs):
    """Builds every node once, in order (so a node used twice is one shared tensor), then reads the outputs
    back last-built first: a read of a late node must not disturb the deferred state of an earlier one."""
    val = {}
    for i, n in enumerate(nodes):
        val[id(n)] = be.from_numpy(inputs[i]) if n.fn is None else n.fn(be, *[val[id(p)] for p in n.parents])
    got = {id(n): be.to_numpy(val[id(n)]) for n in reversed(outs)}
    return [got[id(n)] for n in outs]


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 400))
def test_random_graph_matches_oracle(hip, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    inputs, nodes, outs = random_graph(rng)
    got = evaluate(hip, inputs, nodes, outs)
    ref = evaluate(oracle, inputs, nodes, outs)
    for i, (n, g, e) in enumerate(zip(outs, got, ref)):
        assert g.shape == e.shape == n.shape and g.dtype == e.dtype
        assert np.isfinite(e).all() and np.abs(e).max(initial=0.0) <= n.hi * 1.001, f"seed {seed}: bound of output {i} is wrong"
        np.testing.assert_allclose(g, e, rtol=1e-4, atol=1e-5 * max(1.0, n.hi), err_msg=f"seed {seed} output {i}")


class AsNarrow:
    """A backend seen through a narrow float dtype: f32 arrays go up as their roundings to the dtype, results come back
    widened, and a cast to F32 is a cast to the dtype — so the graphs above run as graphs of that dtype, every op rounding
    its result to it."""

    def __init__(self, be, dt):
        self._be, self._dt = be, dt

    def __getattr__(self, name):
        return getattr(self._be, name)

    def from_numpy(self, arr):
        import cases_fp8
        import cases_half

        arr = np.asarray(arr)
        if arr.dtype != np.float32:
            return self._be.from_numpy(arr)
        if self._dt == A.BF16:
            return self._be.ndarray_from_vec_bf16(cases_half.bf16_round_bits(arr), arr.shape)
        if self._dt == A.F16:
            return self._be.ndarray_from_vec_f16(arr.astype(np.float16), arr.shape)
        return self._be.ndarray_from_vec_fp8(cases_fp8.f8_encode(cases_fp8.f8_round(arr)), arr.shape)

    def to_numpy(self, t):
        import cases_fp8
        import cases_half

        a = self._be.to_numpy(t)
        if a.dtype == np.uint16:
            return cases_half.bf16_widen(a)
        if a.dtype == np.float16:
            return a.astype(np.float32)
        return cases_fp8.f8_decode(a) if a.dtype == np.uint8 else a

    def cast(self, t, dt):
        return self._be.cast(t, self._dt if dt == A.F32 else dt)


@pytest.fixture(scope="module")
def hip_all_narrow():
    """A backend that stores every tensor of a narrow dtype as 2- / 1-byte patterns, however small."""
    from backends import backend_with_env

    be = backend_with_env(CG_NARROW_FROM="2")
    yield be
    be.close()


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 120))
@pytest.mark.parametrize("dt", ["bf16", "f16", "fp8"])
def test_random_graph_in_narrow_dtypes_matches_oracle(hip, hip_all_narrow, oracle, dt, seed):
    """The same random graphs on bf16 / f16 / fp8 tensors, on the default backend (tensors of these sizes are 32-bit
    words) and on one that keeps every tensor as 2- / 1-byte patterns: strided, broadcast, sliced and piecewise views of
    narrow buffers, gathers, row programs and casts over them.  Every op rounds to the dtype on both sides, so exact
    ancestry stays bit-exact; ops whose f32 result may differ in the last place (exp, sin, cos, sums) may differ by one
    unit in the last place of the dtype."""
    code, ulp = {"bf16": (A.BF16, 2.0 ** -8), "f16": (A.F16, 2.0 ** -11), "fp8": (A.F8, 2.0 ** -4)}[dt]
    rng = np.random.default_rng(1000 + seed)
    inputs, nodes, outs = random_graph(rng)
    ref = evaluate(AsNarrow(oracle, code), inputs, nodes, outs)
    for be in (hip, hip_all_narrow):
        got = evaluate(AsNarrow(be, code), inputs, nodes, outs)
        for i, (n, g, e) in enumerate(zip(outs, got, ref)):
            assert g.shape == e.shape == n.shape and g.dtype == e.dtype
            same = (g == e) | (np.isnan(g) & np.isnan(e))
            if n.exact:
                assert same.all(), f"seed {seed} output {i} (exact ancestry)"
            else:
                ok = same | (np.abs(g - e) <= 2 * ulp * np.maximum(np.abs(e), 2.0 ** -6 * max(1.0, n.hi)))
                assert ok.all(), f"seed {seed} output {i}: worst {float(np.nanmax(np.abs(g - e)))}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 200))
def test_random_matmul_shapes_match_oracle(hip, oracle, seed):
    """[.., M, K] x [.., K, N] at random extents, either operand possibly a transposed or sliced view, the
    result possibly consumed by an element-wise op first.  Tolerance: 1e-3 of the result's largest magnitude."""
    rng = np.random.default_rng(5000 + seed)
    big = rng.random() < 0.25
    M, K, N = (int(rng.integers(1, 700 if big else 70)) for _ in range(3))
    if rng.random() < 0.3:
        M = int(rng.integers(1, 9))          # the decode-time row counts
    if rng.random() < 0.3:
        K = int(rng.choice([64, 128, 256, 512]))
    batch = tuple(int(b) for b in rng.integers(1, 4, size=int(rng.integers(0, 3))))
    xt, yt = rng.random() < 0.4, rng.random() < 0.5
    pad = int(rng.integers(0, 5)) if rng.random() < 0.3 else 0
    x = rng.standard_normal(batch + ((K, M) if xt else (M, K + pad))).astype(np.float32)
    y = rng.standard_normal(batch + ((N, K) if yt else (K, N))).astype(np.float32)
    post = str(rng.choice(["none", "scale", "add"]))
    r = len(batch) + 2

    def run(be):
        a, b = be.from_numpy(x), be.from_numpy(y)
        if xt:
            a = be.transpose(a, r - 2, r - 1)
        elif pad:
            a = be.slice(a, r - 1, pad // 2, K)
        if yt:
            b = be.transpose(b, r - 2, r - 1)
        o = be.matmul(a, b)
        if post == "scale":
            o = be.mul(o, const(be, 0.125, o.shape))
        elif post == "add":
            o = be.add(o, o)
        return be.to_numpy(o)

    got, ref = run(hip), run(oracle)
    assert got.shape == ref.shape == batch + (M, N)
    scale = max(1.0, float(np.abs(ref).max()))
    assert float(np.abs(got - ref).max()) <= 1e-3 * scale, f"seed {seed}: M={M} K={K} N={N} batch={batch} xt={xt} yt={yt} pad={pad}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 16))
def test_random_wide_tile_products_match_float64(hip, seed):
    """Products large enough for the 256 x 256 tile (at least 256 tiles), whose loop over k has a lean part (whole tiles of
    aligned operands at fixed per-lane offsets) and a guarded tail: ragged extents in all three directions, either operand
    k-contiguous or row-contiguous (a transposed view), slices that break the 16-byte alignment or leave a row pitch that is
    no multiple of 4, and batches.  Against numpy in float64 (the oracle would take minutes per case); tolerance 1e-3 of
    sum_k |a| |b| per element, as for every product."""
    rng = np.random.default_rng(9100 + seed)
    batch = (2,) if seed % 5 == 4 else ()
    lo = 2900 if batch else 4097
    M, N = (int(rng.integers(lo, lo + 600)) for _ in range(2))
    if seed % 3 == 0:
        M, N = (M + 3) // 4 * 4, (N + 3) // 4 * 4     # multiples of 4: row-contiguous operands take the lean loads too
    K = int(rng.choice([33, 64, 96, 100, 128, 200, 257, 512]))
    xt, yt = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    pad_x, pad_y = (int(rng.choice([0, 0, 1, 4])) for _ in range(2))
    x = (rng.standard_normal(batch + ((K, M + pad_x) if xt else (M, K + pad_x)))).astype(np.float32)
    y = (rng.standard_normal(batch + ((N, K + pad_y) if yt else (K, N + pad_y)))).astype(np.float32)
    r = len(batch) + 2
    a, b = hip.from_numpy(x), hip.from_numpy(y)
    if xt:
        a = hip.transpose(hip.slice(a, r - 1, pad_x, M) if pad_x else a, r - 2, r - 1)
        xv = np.swapaxes(x[..., pad_x:], -1, -2)
    else:
        a = hip.slice(a, r - 1, pad_x, K) if pad_x else a
        xv = x[..., pad_x:]
    if yt:
        b = hip.transpose(hip.slice(b, r - 1, pad_y, K) if pad_y else b, r - 2, r - 1)
        yv = np.swapaxes(y[..., pad_y:], -1, -2)
    else:
        b = hip.slice(b, r - 1, pad_y, N) if pad_y else b
        yv = y[..., pad_y:]
    print(f"seed={seed} batch={batch} M={M} N={N} K={K} xt={xt} yt={yt} pads={pad_x},{pad_y}", flush=True)
    got = hip.to_numpy(hip.matmul(a, b))
    x64, y64 = xv.astype(np.float64), yv.astype(np.float64)
    exact = x64 @ y64
    scale = np.abs(x64) @ np.abs(y64)
    assert got.shape == exact.shape == batch + (M, N)
    err = np.abs(got - exact)
    assert (err <= 1e-3 * scale).all(), f"seed {seed}: worst {float((err / scale).max()):.3e} at {np.unravel_index(np.argmax(err / scale), err.shape)}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 12))
def test_random_wide_tile_products_of_16_bit_dtypes(hip, seed):
    """The same wide tile with bf16 / f16 tensors that cannot take the narrowed-in-memory path (a batch axis, or k no
    multiple of 8): f32 words are narrowed on their way into LDS and multiplied on the 16-bit matrix instructions, with
    either operand k-contiguous or row-contiguous.  Small-integer values: every partial sum is exact in f32, so the result
    must be the rounding of the exact product, bit for bit."""
    import cases_half
    rng = np.random.default_rng(9300 + seed)
    code = A.BF16 if seed % 2 == 0 else A.F16
    batch = (2,) if seed % 3 != 2 else ()
    lo = 2900 if batch else 4097
    M, N = (int(rng.integers(lo, lo + 300)) for _ in range(2))
    if seed % 4 == 1:
        M, N = (M + 3) // 4 * 4, (N + 3) // 4 * 4
    K = int(rng.choice([96, 130, 200, 264])) if batch else int(rng.choice([100, 130, 203]))
    xt, yt = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
    xv = rng.integers(-6, 7, size=batch + (M, K)).astype(np.float32)
    yv = rng.integers(-6, 7, size=batch + (K, N)).astype(np.float32)
    r = len(batch) + 2
    up = lambda v: cases_half.from_half(hip, code, cases_half.round_to(code, np.ascontiguousarray(v)))
    a = hip.transpose(up(np.swapaxes(xv, -1, -2)), r - 2, r - 1) if xt else up(xv)
    b = hip.transpose(up(np.swapaxes(yv, -1, -2)), r - 2, r - 1) if yt else up(yv)
    print(f"seed={seed} dtype={'bf16' if code == A.BF16 else 'f16'} batch={batch} M={M} N={N} K={K} xt={xt} yt={yt}", flush=True)
    got = cases_half.as_f32(code, cases_half.read(hip, hip.matmul(a, b)))
    exact = (xv.astype(np.float64) @ yv.astype(np.float64)).astype(np.float32)
    exp = cases_half.as_f32(code, cases_half.round_to(code, exact))
    bad = np.argwhere(got != exp)
    assert bad.size == 0, f"seed {seed}: {len(bad)} mismatches, first {bad[:3].tolist()}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 18))
def test_random_products_of_operands_that_lie_narrow(hip, seed):
    """Products of bf16 / f16 / fp8 tensors that lie in memory as 2- / 1-byte patterns (uploads of 65536 elements and
    more): big ones (the 256 x 256 tile of narrow operands) and few-row ones (a decode-time linear layer), with the
    operands whole — multiplied as they lie —, or cut by slices that move the first element off a 16-byte boundary, leave
    a row pitch that is no multiple of 16 bytes or take a window of the rows (then narrowed or widened first), or
    transposed so that k is not contiguous.  Small-integer values: every partial sum is exact in f32, so the result must
    be the rounding of the exact product, bit for bit."""
    import cases_fp8
    import cases_half

    rng = np.random.default_rng(9300 + seed)
    dt = ("bf16", "f16", "fp8")[seed % 3]
    few = seed % 2 == 1
    M = int(rng.integers(1, 9)) if few else int(rng.integers(4097, 4400))
    N = int(rng.integers(300, 2000)) if few else int(rng.integers(4097, 4400))
    K = int(rng.choice([256, 512, 1024, 2048])) if few else int(rng.choice([64, 128, 192, 256]))
    row_pad = int(rng.choice([0, 0, 8, 16, 3]))         # extra columns in the weight's rows (a slice takes K of them)
    col_off = int(rng.choice([0, 0, 8, 16, 1])) if row_pad else 0
    col_off = min(col_off, row_pad)
    row_off = int(rng.choice([0, 0, 5, 64]))             # rows skipped at the top of the weight
    yt = bool(rng.random() < 0.2)                         # the weight as [K, N] (k not contiguous)
    lim = 3 if dt == "fp8" else 6
    xv = rng.integers(-lim, lim + 1, size=(M, K)).astype(np.float32)
    wv = rng.integers(-lim, lim + 1, size=(N + row_off, K + row_pad)).astype(np.float32)

    def up(v):
        v = np.ascontiguousarray(v)
        if dt == "fp8":
            return hip.ndarray_from_vec_fp8(cases_fp8.f8_encode(v), v.shape)
        code = A.BF16 if dt == "bf16" else A.F16
        return cases_half.from_half(hip, code, cases_half.round_to(code, v))

    a = up(xv)
    if yt:
        b = up(np.ascontiguousarray(wv[row_off:, col_off:col_off + K].T))
    else:
        w = up(wv)
        if row_off:
            w = hip.slice(w, 0, row_off, N)
        if row_pad:
            w = hip.slice(w, 1, col_off, K)
        b = hip.transpose(w, 0, 1)
    print(f"seed={seed} dtype={dt} M={M} N={N} K={K} row_pad={row_pad} col_off={col_off} row_off={row_off} yt={yt}", flush=True)
    got = hip.to_numpy(hip.matmul(a, b))
    exact = (xv.astype(np.float64) @ wv[row_off:, col_off:col_off + K].astype(np.float64).T).astype(np.float32)
    if dt == "fp8":
        got, exp = cases_fp8.f8_decode(got), cases_fp8.f8_round(exact)
    else:
        code = A.BF16 if dt == "bf16" else A.F16
        got, exp = cases_half.as_f32(code, got), cases_half.as_f32(code, cases_half.round_to(code, exact))
    bad = np.argwhere(got != exp)
    assert bad.size == 0, f"seed {seed}: {len(bad)} mismatches, first {bad[:3].tolist()}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 12))
def test_random_products_through_the_lds_ring(hip, seed):
    """Big products of narrow operands whose rows of k are whole turns of the four-stage LDS ring (random multiples of 128
    values of the 16-bit dtypes, of 256 of fp8): the kernel whose workgroups walk the tiles, at random extents (ragged
    tiles, more or fewer tiles than four rounds), with a result width that is a multiple of 4 (rounded in the product's
    store) or not (f32 result and the rounding pass), the weight whole or as a window of wider rows.  Small integers: the
    rounding of the exact product, bit for bit."""
    import cases_fp8
    import cases_half

    rng = np.random.default_rng(9400 + seed)
    dt = ("bf16", "f16", "fp8")[seed % 3]
    M = int(rng.integers(3600, 5200))
    N = int(rng.integers(3600, 5200))
    if seed % 2 == 0:
        N -= N % 4
    if M * N < 256 * 65536 + 300000:       # (at least 256 tiles of 256 x 256)
        M = 4200
    K = (256 * int(rng.integers(1, 5))) if dt == "fp8" else (128 * int(rng.integers(1, 11)))
    row_pad = int(rng.choice([0, 0, 16, 32]))
    col_off = int(rng.choice([0, 16])) if row_pad else 0
    col_off = min(col_off, row_pad)
    lim = 3 if dt == "fp8" else 6
    xv = rng.integers(-lim, lim + 1, size=(M, K)).astype(np.float32)
    wv = rng.integers(-lim, lim + 1, size=(N, K + row_pad)).astype(np.float32)
    if dt == "fp8":
        wv *= (rng.random(wv.shape) < 0.25)        # (sums stay small enough for fp8's few exact integers to matter)

    def up(v):
        v = np.ascontiguousarray(v)
        if dt == "fp8":
            return hip.ndarray_from_vec_fp8(cases_fp8.f8_encode(v), v.shape)
        code = A.BF16 if dt == "bf16" else A.F16
        return cases_half.from_half(hip, code, cases_half.round_to(code, v))

    w = up(wv)
    if row_pad:
        w = hip.slice(w, 1, col_off, K)
    print(f"seed={seed} dtype={dt} M={M} N={N} K={K} row_pad={row_pad} col_off={col_off}", flush=True)
    got = hip.to_numpy(hip.matmul(up(xv), hip.transpose(w, 0, 1)))
    exact = xv @ wv[:, col_off:col_off + K].T          # (sgemm on small integers: exact)
    assert np.abs(exact).max() < 2 ** 24
    if dt == "fp8":
        got, exp = cases_fp8.f8_decode(got), cases_fp8.f8_round(exact)
    else:
        code = A.BF16 if dt == "bf16" else A.F16
        got, exp = cases_half.as_f32(code, got), cases_half.as_f32(code, cases_half.round_to(code, exact))
    bad = np.argwhere(got != exp)
    assert bad.size == 0, f"seed {seed}: {len(bad)} mismatches, first {bad[:3].tolist()}"


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 120))
def test_random_attention_shapes_match_oracle(hip, oracle, seed):
    """The model graphs' attention (repeat_kv, scores, scale, causal mask rows, soft-max, context) at random
    batch / head / query / cache extents: decode steps (one query), speculative-width chunks and prefill chunks
    that start anywhere in the cache, head widths with and without a one-pass kernel."""
    import cases

    rng = np.random.default_rng(9000 + seed)
    B, kvh, rep = int(rng.integers(1, 3)), int(rng.integers(1, 4)), int(rng.choice([1, 2, 4, 8]))
    hd = int(rng.choice([64, 64, 128, 128, 32, 80]))
    T = int(rng.integers(1, 600))
    S = int(rng.choice([1, 1, int(rng.integers(1, 10)), int(rng.integers(1, T + 1)), T]))
    S = min(S, T)
    q = rng.standard_normal((B, kvh * rep, S, hd)).astype(np.float32)
    k = rng.standard_normal((B, kvh, T, hd)).astype(np.float32)
    v = rng.standard_normal((B, kvh, T, hd)).astype(np.float32)

    def run(be):
        return be.to_numpy(cases.decode_attention_ops(be, be.from_numpy(q), be.from_numpy(k), be.from_numpy(v), rep))

    got, ref = run(hip), run(oracle)
    assert got.shape == ref.shape == (B, kvh * rep, S, hd)
    np.testing.assert_allclose(got, ref, rtol=1e-4, atol=2e-5, err_msg=f"seed {seed}: B={B} kvh={kvh} rep={rep} hd={hd} S={S} T={T}")


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 28))
def test_random_decoder_blocks_match_oracle(hip, oracle, seed):
    """The dense part of a decoder layer at decode time (residual add in the store of the o / down product, RMS norm in
    the loads of the products behind it, gated pair) with random row counts and widths, and with the results — norms and
    raw products included or not — read back in a random order, which decides what is still deferred when each
    product runs.  1e-3 of the values' scale (they are of order one)."""
    import cases

    rng = np.random.default_rng(7000 + seed)
    B = int(rng.integers(1, 6))
    if seed < 12:
        H = int(rng.choice([2048, 2048, 4096, 1024, 3072, 512]))
        F = int(rng.choice([4096, 6144, 8192]))
        kv = int(rng.choice([256, 512, 2048]))
    else:   # widths that are no multiples of 1024 (ragged chunks of k, few columns)
        H = int(rng.choice([576, 640, 960, 1536, 2560, 260, 1028]))
        F = int(rng.choice([1536, 2560, 6912, 1540, 512]))
        kv = int(rng.choice([192, 320, 576, 128]))
    sc = np.float32(1.0 / np.sqrt(H))
    r = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    x0, a0 = r(B, 1, H), r(B, 1, H)
    wo, wg, wu, wd = r(H, H) * sc, r(F, H) * sc, r(F, H) * sc, r(H, F) * np.float32(1.0 / np.sqrt(F))
    wq, wk, wv = r(H, H) * sc, r(kv, H) * sc, r(kv, H) * sc
    g1, g2 = 1 + 0.1 * r(H), 1 + 0.1 * r(H)
    wanted = ["q", "k", "v", "h1", "h2"] + [n for n in ("n1", "n2", "g", "u", "act") if rng.random() < 0.35]
    order = [wanted[i] for i in rng.permutation(len(wanted))]
    two_norm_uses = rng.random() < 0.5      # the second norm also feeds an element-wise op

    def run(be):
        shp, fs = (B, 1, H), (B, 1, F)
        L, C = cases._linear, cases._const
        t = {}
        t["h1"] = be.add(be.from_numpy(x0).move(), L(be, be.from_numpy(a0), be.from_numpy(wo)).move())
        t["n1"] = cases._rmsnorm_ops(be, t["h1"], be.from_numpy(g1), H, shp)
        t["g"], t["u"] = L(be, t["n1"], be.from_numpy(wg)), L(be, t["n1"], be.from_numpy(wu))
        e = be.exp(be.neg(t["g"]).move())
        sg = be.div(C(be, 1.0, fs).move(), be.add(C(be, 1.0, fs).move(), e.move()).move())
        t["act"] = be.mul(be.mul(t["g"], sg.move()).move(), t["u"])
        t["h2"] = be.add(t["h1"], L(be, t["act"], be.from_numpy(wd)).move())
        t["n2"] = cases._rmsnorm_ops(be, t["h2"], be.from_numpy(g2), H, shp)
        t["q"], t["k"], t["v"] = (L(be, t["n2"], be.from_numpy(w)) for w in (wq, wk, wv))
        extra = be.to_numpy(be.add(t["n2"], t["n2"])) if two_norm_uses else None
        for name in list(t):
            if name not in order:
                del t[name]
        outs = {name: be.to_numpy(t[name]) for name in order}
        return outs, extra

    got, gx = run(hip)
    ref, rx = run(oracle)
    for name in order:
        assert got[name].shape == ref[name].shape
        err = float(np.abs(got[name].astype(np.float64) - ref[name]).max())
        assert err <= 1e-3 * max(4.0, float(np.abs(ref[name]).max())), f"seed {seed} B={B} H={H} F={F} kv={kv} {name} order={order}: {err}"
    if two_norm_uses:
        np.testing.assert_allclose(gx, rx, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("seed", range(SEED0, SEED0 + 48))
def test_random_attention_block_steps_match_oracle(hip, oracle, seed):
    """Decode steps of a whole attention block (q / k / v projections, heads split off, rotary embedding, cache append,
    attention) at random row counts, widths, head counts and sizes and cache lengths, with or without an RMS norm of a
    residual stream in front, and with random extra holders of the intermediate handles (a clone of a projection or of
    a roped tensor that is read later, the roped q read back before the attention): who else holds a product decides
    whether the embedding and the append may run in the products' store.  From seed 24 on: hidden sizes that are no
    multiples of 1024, and (half of them) an RMS norm per head on q and k between the projection and the embedding, as in
    the Qwen3 block, with random holders of the normed tensors too.  1e-3 of the values' scale (order one)."""
    import cases

    rng = np.random.default_rng(11000 + seed)
    B = int(rng.integers(1, 6))
    K = int(rng.choice([1024, 2048, 2048, 3072, 512])) if seed < 24 else int(rng.choice([576, 1024, 1024, 960, 1536, 640, 2048, 2560, 4096]))
    hd = int(rng.choice([64, 64, 128, 32]))
    qk = seed >= 24 and bool(rng.random() < 0.6)
    kvh, rep = int(rng.integers(1, 5)), int(rng.choice([1, 2, 4]))
    H = kvh * rep
    T = int(rng.choice([int(rng.integers(1, 40)), int(rng.integers(200, 700)), int(rng.integers(1000, 2300))]))
    steps = int(rng.integers(1, 4))
    normed = bool(rng.random() < 0.5)
    keep = {n: bool(rng.random() < 0.2) for n in ("q_raw", "k_raw", "v_raw", "q_rope", "k_rope")}
    keep.update({n: qk and bool(rng.random() < 0.15) for n in ("q_norm", "k_norm")})
    read_q_first = bool(rng.random() < 0.25)
    sc = np.float32(1.0 / np.sqrt(K))
    r = lambda *s: rng.standard_normal(s).astype(np.float32)  # noqa: E731
    xs, res = [r(B, 1, K) for _ in range(steps)], [r(B, 1, K) for _ in range(steps)]
    wo, gm = r(K, K) * sc, (1 + 0.1 * r(K)).astype(np.float32)
    wq, wk, wv = r(H * hd, K) * sc, r(kvh * hd, K) * sc, r(kvh * hd, K) * sc
    ck, cv = r(B, kvh, T, hd), r(B, kvh, T, hd)
    ang = rng.uniform(0, 6.28, (T + steps, hd)).astype(np.float32)
    cos_t, sin_t = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    gq, gk = (1 + 0.1 * r(hd)).astype(np.float32), (1 + 0.1 * r(hd)).astype(np.float32)

    def run(be):
        k_cache, v_cache = be.from_numpy(ck), be.from_numpy(cv)
        tcos, tsin = be.from_numpy(cos_t), be.from_numpy(sin_t)
        weights = [be.from_numpy(w) for w in (wq, wk, wv)]
        outs = []
        for step in range(steps):
            pos = T + step
            held = {}
            if normed:
                h = be.add(be.from_numpy(res[step]).move(), cases._linear(be, be.from_numpy(xs[step]), be.from_numpy(wo)).move())
                xn = cases._rmsnorm_ops(be, h, be.from_numpy(gm), K, (B, 1, K))
                del h
            else:
                xn = be.from_numpy(xs[step])
            q, k, v = (cases._linear(be, xn, w) for w in weights)
            del xn
            for name, t in (("q_raw", q), ("k_raw", k), ("v_raw", v)):
                if keep[name]:
                    held[name] = t.clone()

            def heads(t, n):
                return be.transpose(be.reshape(t.move(), (B, 1, n, hd)).move(), 1, 2)

            def rope(t, n):
                sh = (B, n, 1, hd)
                c = be.broadcast(be.reshape(be.slice(tcos, 0, pos, 1).move(), (1, 1, 1, hd)).move(), sh)
                s_ = be.broadcast(be.reshape(be.slice(tsin, 0, pos, 1).move(), (1, 1, 1, hd)).move(), sh)
                rot = cases._rot_half(be, t, hd // 2)
                return be.add(be.mul(c.move(), t.move()).move(), be.mul(s_.move(), rot.move()).move())

            q, k, v = heads(q, H), heads(k, kvh), heads(v, kvh)
            if qk:
                def head_norm(t, n, g):
                    flat = be.reshape(t.move(), (B * n, hd))
                    nt = cases._rmsnorm_ops(be, flat, be.from_numpy(g), hd, (B * n, hd))
                    del flat
                    return be.reshape(nt.move(), (B, n, 1, hd))

                q, k = head_norm(q, H, gq), head_norm(k, kvh, gk)
                if keep["q_norm"]:
                    held["q_norm"] = q.clone()
                if keep["k_norm"]:
                    held["k_norm"] = k.clone()
            q, k = rope(q, H), rope(k, kvh)
            if keep["q_rope"]:
                held["q_rope"] = q.clone()
            if keep["k_rope"]:
                held["k_rope"] = k.clone()
            k_cache = be.concat(k_cache.move(), k.move(), 2)
            v_cache = be.concat(v_cache.move(), v.move(), 2)
            if read_q_first:
                outs.append(be.to_numpy(q))
            outs.append(be.to_numpy(cases.decode_attention_ops(be, q, k_cache.clone(), v_cache.clone(), rep)))
            outs += [be.to_numpy(be.slice(k_cache, 2, pos, 1)), be.to_numpy(be.slice(v_cache, 2, pos, 1))]
            outs += [be.to_numpy(held[n]) for n in sorted(held)]
        outs.append(be.to_numpy(k_cache))
        return outs

    got, ref = run(hip), run(oracle)
    assert len(got) == len(ref)
    what = f"seed {seed}: B={B} K={K} hd={hd} kvh={kvh} rep={rep} T={T} steps={steps} normed={normed} qk={qk} keep={keep} read_q_first={read_q_first}"
    for i, (g, e) in enumerate(zip(got, ref)):
        assert g.shape == e.shape, what
        err = float(np.abs(g.astype(np.float64) - e).max())
        assert err <= 1e-3 * max(4.0, float(np.abs(e).max())), f"{what} output {i}: {err}"

"""Operands of the products of the 16-bit dtypes: a tensor that lies in memory as 2-byte patterns is multiplied as it
lies (no copy is made); one that lies there as 32-bit words (CG_NARROW_STORAGE=0, small tensors, results of kernels that
store words) gets a narrow copy that is kept with its buffer, one per view that was multiplied: several slices of one
weight buffer each keep theirs, and a copy never outlives a write into its buffer."""
import numpy as np
import pytest

from catgrad_amd import _abi as A
from cases_half import as_f32, bf16_values, from_half, read

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", params=["narrow", "words"])
def hipm(request):
    """(backend, True when its tensors of narrow dtypes lie in memory as 32-bit words)."""
    from backends import backend_with_env

    be = backend_with_env(CG_NARROW_STORAGE="0" if request.param == "words" else "1")
    yield be, request.param == "words"
    be.close()


def _tol(ref):
    return 2.0 ** -8 * np.abs(ref) + 1e-3 * np.abs(ref).max()   # one bf16 unit in the last place + the reduction tolerance


def test_three_slices_of_one_weight_buffer_are_narrowed_once_each(hipm, oracle):
    """A fused q/k/v weight [3 * 1024, 2048] multiplied slice by slice by four decode-time rows, twice.  Held as 32-bit
    words: three narrowing launches in all (one per slice, kept with the buffer for the second round); held as bf16
    patterns: none.  Results equal to the oracle's either way."""
    hip, words = hipm
    dt = A.BF16
    ux, x = bf16_values(7001, (4, 1, 2048), 0.25)
    uw, w = bf16_values(7002, (3 * 1024, 2048), 0.25)

    def products(be, rounds):
        tw = from_half(be, dt, uw)
        outs = []
        for _ in range(rounds):
            tx = from_half(be, dt, ux)
            for s in range(3):
                ws = be.slice(tw, 0, s * 1024, 1024)
                wv = be.broadcast(be.transpose(ws, 0, 1), (4, 2048, 1024))
                outs.append(as_f32(dt, read(be, be.matmul(tx, wv))))
        return outs

    hip.profile_enable(A.K_PACK, 1)
    hip.profile_read(A.K_PACK, reset=True)
    got = products(hip, 2)
    packs = hip.profile_read(A.K_PACK, reset=True)[0]
    hip.profile_enable(A.K_PACK, 0)
    assert packs == (3 if words else 0), packs
    exp = products(oracle, 1)
    ref64 = x.astype(np.float64)[:, 0] @ w.astype(np.float64).T
    for i, g in enumerate(got):
        s = i % 3
        r = ref64[:, s * 1024:(s + 1) * 1024]
        assert np.all(np.abs(g[:, 0] - r) <= _tol(r)), i
        assert np.all(np.abs(g[:, 0] - exp[s][:, 0]) <= _tol(r)), i


def test_two_slices_of_one_weight_buffer_in_big_products(hipm, oracle):
    """The same with products big enough for the 256 x 256 tile of narrow operands (4096 x 2048 x 4096, twice per round).
    Held as words: the two weight slices are narrowed once each; the activations, which the caller holds across the two
    products of a round, once per round.  Held as bf16 patterns: both operands are multiplied as they lie."""
    hip, words = hipm
    dt = A.BF16
    ux, x = bf16_values(7003, (1, 4096, 2048), 0.25)
    uw, w = bf16_values(7004, (2 * 4096, 2048), 0.25)

    def products(be, rounds):
        tw = from_half(be, dt, uw)
        outs = []
        for _ in range(rounds):
            tx = from_half(be, dt, ux)
            for s in range(2):
                ws = be.slice(tw, 0, s * 4096, 4096)
                wv = be.broadcast(be.transpose(ws, 0, 1), (1, 2048, 4096))
                outs.append(as_f32(dt, read(be, be.matmul(tx, wv))))
        return outs

    hip.profile_enable(A.K_PACK, 1)
    hip.profile_read(A.K_PACK, reset=True)
    got = products(hip, 2)
    packs = hip.profile_read(A.K_PACK, reset=True)[0]
    hip.profile_enable(A.K_PACK, 0)
    assert packs == (2 + 2 if words else 0), packs
    ref64 = x.astype(np.float64)[0] @ w.astype(np.float64).T
    for i, g in enumerate(got):
        r = ref64[:, (i % 2) * 4096:(i % 2 + 1) * 4096]
        assert np.all(np.abs(g[0] - r) <= _tol(r)), i


def test_a_narrow_copy_does_not_outlive_an_in_place_append(hipm, oracle):
    """x . w, then rows appended to w's buffer in place (a stack growing along its outermost axis), then the product
    with the grown matrix and with a window of it that starts inside the old rows: the copy kept for the first product
    is dropped by the append and never read again.  (A stack that may grow holds 32-bit words in either mode.)"""
    hip, words = hipm
    dt = A.BF16
    ux, x = bf16_values(7011, (4096, 2048), 0.25)
    uw1, w1 = bf16_values(7012, (2048, 2048), 0.25)
    uw2, w2 = bf16_values(7013, (2048, 2048), 0.25)
    uw3, w3 = bf16_values(7014, (256, 2048), 0.25)

    def run(be):
        tx = from_half(be, dt, ux)
        stack = be.concat(from_half(be, dt, uw1), from_half(be, dt, uw2), 0)    # a fresh buffer with room to grow
        first = as_f32(dt, read(be, be.matmul(tx, be.transpose(stack, 0, 1))))   # narrows the [4096, 2048] view
        grown = be.concat(stack, from_half(be, dt, uw3), 0)                      # uniquely held: appended in place
        del stack
        second = as_f32(dt, read(be, be.matmul(tx, be.transpose(grown, 0, 1))))
        window = as_f32(dt, read(be, be.matmul(tx, be.transpose(be.slice(grown, 0, 256, 4096), 0, 1))))
        return first, second, window

    g1, g2, g3 = run(hip)
    wall = np.concatenate([w1, w2, w3]).astype(np.float64)
    r = x.astype(np.float64) @ wall.T
    for g, ref in ((g1, r[:, :4096]), (g2, r), (g3, r[:, 256:])):
        assert g.shape == ref.shape
        assert np.all(np.abs(g - ref) <= _tol(ref))
    e1, e2, e3 = run(oracle)
    for g, e in ((g1, e1), (g2, e2), (g3, e3)):
        assert np.all(np.abs(g - e) <= _tol(r).max())

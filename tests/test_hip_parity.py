"""Parity tests proper: HipBackend (through the C ABI) against the CPU oracle on the
same seeded inputs, and against the reference's known answers.

Tolerances (written out in cases.assert_close): bit-exact for integer / shape / index
ops and IEEE-exact f32 ops; rtol 1e-4 (+1e-6 abs) for f32 element-wise math; 1e-3 of
the natural scale for matmul and sum."""
import numpy as np
import pytest

from catgrad_amd import BackendPanic, ShapeError
from catgrad_amd import _abi as A
from cases import CASES, assert_close
from kat_runner import KATS, apply, check_case

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("case", CASES, ids=lambda c: c.name)
def test_hip_matches_oracle(hip, oracle, case):
    print(f"case={case.name}", flush=True)
    got = case.run(hip)
    ref = case.run(oracle)
    scales = case.scale() if case.scale else [None] * len(ref)
    assert len(got) == len(ref)
    for i, (g, e, s) in enumerate(zip(got, ref, scales)):
        assert g.dtype == e.dtype
        assert_close(case.kind, g, e, s, f"{case.name}[{i}]")


@pytest.mark.parametrize("case", [c for c in CASES if c.expect is not None], ids=lambda c: c.name)
def test_hip_matches_closed_form(hip, case):
    print(f"case={case.name}", flush=True)
    got = case.run(hip)
    exp = case.expect()
    scales = case.scale() if case.scale else [None] * len(exp)
    for i, (g, e, s) in enumerate(zip(got, exp, scales)):
        assert_close(case.kind, g, e, s, f"{case.name}[{i}]")


@pytest.fixture(scope="module")
def hip_segments():
    """A backend whose decode-time attention always takes the workgroup-per-(KV head, segment) kernel (by default only
    long caches do): CG_ATTN_SEG_FROM is read when a backend is created."""
    import os

    from catgrad_amd import HipBackend

    old = os.environ.get("CG_ATTN_SEG_FROM")
    os.environ["CG_ATTN_SEG_FROM"] = "1"
    try:
        be = HipBackend(0)
    finally:
        if old is None:
            del os.environ["CG_ATTN_SEG_FROM"]
        else:
            os.environ["CG_ATTN_SEG_FROM"] = old
    yield be
    be.close()


@pytest.mark.parametrize("case", [c for c in CASES if c.name.startswith(("decode_attention_", "decode_qkv_rope_append_"))],
                         ids=lambda c: c.name)
def test_segment_attention_kernel_matches_closed_form_and_oracle(hip_segments, oracle, case):
    print(f"case={case.name} (segment kernel)", flush=True)
    got = case.run(hip_segments)
    exp = case.expect()
    ref = case.run(oracle)
    scales = case.scale() if case.scale else [None] * len(exp)
    for i, (g, e, r, s) in enumerate(zip(got, exp, ref, scales)):
        assert_close(case.kind, g, e, s, f"{case.name}[{i}] vs closed form")
        assert_close(case.kind, g, r, s, f"{case.name}[{i}] vs oracle")


@pytest.fixture(scope="module")
def hip_narrow_everywhere():
    """A backend that keeps EVERY tensor of a narrow float dtype as 2- / 1-byte patterns (by default only tensors of 65536
    elements and more): the small tensors of the 16-bit and fp8 cases then take the narrow-format loads and stores of every
    kernel, the widened copies of the kernels that address words, and the declines of the decode-time fusions."""
    from backends import backend_with_env

    be = backend_with_env(CG_NARROW_FROM="2")
    yield be
    be.close()


@pytest.fixture(scope="module")
def hip_words_only():
    """A backend that keeps tensors of the narrow float dtypes as 32-bit words (CG_NARROW_STORAGE=0)."""
    from backends import backend_with_env

    be = backend_with_env(CG_NARROW_STORAGE="0")
    yield be
    be.close()


@pytest.mark.parametrize("case", [c for c in CASES if c.name.startswith(("half_", "fp8_"))], ids=lambda c: c.name)
def test_narrow_storage_of_small_tensors_matches_oracle(hip_narrow_everywhere, hip_words_only, oracle, case):
    print(f"case={case.name} (narrow storage from 2 elements)", flush=True)
    got = case.run(hip_narrow_everywhere)
    wide = case.run(hip_words_only)
    ref = case.run(oracle)
    scales = case.scale() if case.scale else [None] * len(ref)
    assert len(got) == len(ref) == len(wide)
    for i, (g, w, e, s) in enumerate(zip(got, wide, ref, scales)):
        assert g.dtype == e.dtype
        assert_close(case.kind, g, e, s, f"{case.name}[{i}]")
        assert_close(case.kind, w, e, s, f"{case.name}[{i}] (32-bit words)")
    if case.expect is not None:
        for i, (g, e, s) in enumerate(zip(got, case.expect(), scales)):
            assert_close(case.kind, g, e, s, f"{case.name}[{i}] vs closed form")


def test_narrow_tensors_occupy_their_own_width(hip, oracle):
    """A bf16 tensor of 8192 x 8192 and an fp8 tensor of the same shape take 128 and 64 MiB of device memory; the sum
    and the product of two such tensors, a strided view, a concat, a gather and a row sum of them are stored / computed
    as the oracle does, and nothing but the pool's rounding is held afterwards."""
    import cases_fp8
    import cases_half

    hip.sync()
    hip.pool_trim()
    base = hip.pool_stats()[0]
    n = 8192
    ua, a = cases_half.bf16_values(9101, (n, n), 1.0)
    ub, b = cases_half.bf16_values(9102, (n, n), 1.0)
    ta, tb = cases_half.from_half(hip, A.BF16, ua), cases_half.from_half(hip, A.BF16, ub)
    held = hip.pool_stats()[0] - base
    assert 2 * n * n * 2 <= held <= 2 * n * n * 2 + (64 << 20), held          # 2 bytes per element (+ size classes)
    tsum = hip.add(ta, tb)
    got = cases_half.as_f32(A.BF16, cases_half.read(hip, tsum))
    exp = cases_half.as_f32(A.BF16, cases_half.round_to(A.BF16, a + b))
    assert np.array_equal(got, exp)
    held = hip.pool_stats()[0] - base
    assert held <= 3 * n * n * 2 + (96 << 20), held                           # the sum is stored narrow as well
    # a strided view (every other row, transposed) materialised by reshape; a row sum; a gather of rows
    view = hip.reshape(hip.transpose(hip.slice(tsum, 0, 1, n - 1), 0, 1), (n * (n - 1),))
    got = cases_half.as_f32(A.BF16, cases_half.read(hip, view))
    assert np.array_equal(got, exp[1:].T.reshape(-1))
    del view
    rows = cases_half.as_f32(A.BF16, cases_half.read(hip, hip.sum(tsum)))
    ref = exp.astype(np.float64).sum(-1, keepdims=True)
    assert np.all(np.abs(rows - ref) <= 2.0 ** -7 * np.abs(ref) + 1e-3 * np.abs(exp).sum(-1, keepdims=True))
    idx = np.array([5, 8191, 0, 5, 4096], np.uint32)
    few = cases_half.as_f32(A.BF16, cases_half.read(hip, hip.index(tsum, 0, hip.from_numpy(idx))))
    assert np.array_equal(few, exp[idx])
    many = np.arange(0, n, 3, dtype=np.uint32)[::-1].copy()
    big = cases_half.as_f32(A.BF16, cases_half.read(hip, hip.index(tsum, 0, hip.from_numpy(many))))
    assert np.array_equal(big, exp[many])
    cols = cases_half.as_f32(A.BF16, cases_half.read(hip, hip.index(tsum, 1, hip.from_numpy(idx))))
    assert np.array_equal(cols, exp[:, idx])
    cat = cases_half.as_f32(A.BF16, cases_half.read(hip, hip.concat(hip.slice(tsum, 1, 0, 100), hip.slice(ta, 1, 7, 33), 1)))
    assert np.array_equal(cat, np.concatenate([exp[:, :100], a[:, 7:40]], 1))
    del tsum, ta, tb
    # fp8: 1 byte per element
    rng = np.random.default_rng(9103)
    codes = rng.integers(0, 256, (n, n), dtype=np.uint8)
    codes[(codes & 0x7F) == 0x7F] = 0x38                                        # no NaNs: 1.0 instead
    t8 = hip.ndarray_from_vec_fp8(codes, codes.shape)
    held = hip.pool_stats()[0] - base
    assert n * n <= held <= n * n + (32 << 20), held
    back = hip.to_numpy(hip.reshape(hip.transpose(t8, 0, 1), (n * n,)))
    assert back.dtype == np.uint8 and np.array_equal(back.reshape(n, n), codes.T)
    del t8
    hip.sync()
    hip.pool_trim()
    assert hip.pool_stats()[0] - base <= (1 << 20)


@pytest.mark.parametrize("case", KATS["cases"], ids=lambda c: c["name"])
def test_hip_reference_kat(hip, case):
    check_case(hip, case)


@pytest.mark.parametrize("case", KATS["errors"], ids=lambda c: c["name"])
def test_hip_reference_error(hip, case):
    with pytest.raises(BackendPanic) as e:
        apply(hip, case)
    if "message" in case:
        assert case["message"] in str(e.value)


def test_from_vec_shape_error(hip):
    with pytest.raises(ShapeError):
        hip.ndarray_from_vec_f32([1.0, 2.0, 3.0], (2, 2))
    with pytest.raises(ShapeError):
        hip.ndarray_from_vec_u32([1, 2, 3, 4], (3,))


def test_error_paths(hip):
    x = hip.from_numpy(np.arange(12, dtype=np.float32).reshape(3, 4))
    u = hip.from_numpy(np.arange(12, dtype=np.uint32).reshape(3, 4))
    for bad in (
        lambda: hip.add(x, u),
        lambda: hip.sin(u),
        lambda: hip.topk(u, 2),
        lambda: hip.topk(x, 5),
        lambda: hip.matmul(x, x),
        lambda: hip.matmul(x, hip.reshape(x, (1, 4, 3))),
        lambda: hip.slice(x, 1, 3, 2),
        lambda: hip.slice(x, 2, 0, 1),
        lambda: hip.transpose(x, 0, 2),
        lambda: hip.reshape(x, (5, 2)),
        lambda: hip.concat(x, hip.reshape(x, (4, 3)), 0),
        lambda: hip.index(x, 0, x),
        lambda: hip.max(hip.from_numpy(np.float32(1).reshape(()))),
        lambda: hip.argmax(hip.zeros((3, 0), A.F32)),
        lambda: hip.zeros((2, 2), 9),            # not a dtype
        lambda: hip.cast(x, 9),
        lambda: hip.add(hip.cast(x, A.F8), hip.cast(x, A.BF16)),
        lambda: hip.add(hip.cast(x, A.F16), hip.cast(x, A.BF16)),
        lambda: hip.matmul(hip.cast(x, A.F16), hip.transpose(x, 0, 1)),
        lambda: hip.div(hip.broadcast(hip.from_numpy(np.uint32(3).reshape(())), (2,)),
                        hip.zeros((2,), A.U32)),
    ):
        with pytest.raises(BackendPanic):
            bad()


def test_deferred_device_faults(hip):
    """Gather index out of range and u32 division by zero are detected by the kernel and
    reported by the next call that waits for the device (the reference panics at once)."""
    w = hip.from_numpy(np.arange(20, dtype=np.float32).reshape(5, 4))
    bad = hip.index(w, 0, hip.from_numpy(np.array([1, 7], np.uint32)))
    with pytest.raises(BackendPanic, match="out of bounds"):
        hip.sync()
    np.testing.assert_array_equal(hip.to_numpy(bad)[0], np.arange(4, 8, dtype=np.float32))
    a = hip.from_numpy(np.array([4, 6, 8], np.uint32))
    q = hip.div(a, hip.from_numpy(np.array([2, 0, 4], np.uint32)))
    with pytest.raises(BackendPanic, match="divide by zero"):
        hip.to_vec(q)
    hip.sync()  # the fault word was cleared


def test_clone_is_refcount_and_values_survive_release(hip):
    x = hip.from_numpy(np.arange(6, dtype=np.float32).reshape(2, 3))
    y = x.clone()
    t = hip.transpose(x.move(), 0, 1)
    del y
    np.testing.assert_array_equal(hip.to_numpy(t), np.arange(6, dtype=np.float32).reshape(2, 3).T)


def test_pool_returns_to_baseline(hip):
    hip.sync()
    base, _ = hip.pool_stats()
    for _ in range(3):
        a = hip.from_numpy(np.ones((257, 129), np.float32))
        b = hip.exp(hip.add(a, a))
        c = hip.sum(b)
        hip.to_numpy(c)
        del a, b, c
    now, cached = hip.pool_stats()
    assert now == base
    assert cached > 0


def test_decode_attention_runs_as_one_fused_pass(hip):
    """The decode-step attention graph (head_dim 64, 4 query heads per KV head) is absorbed by the fused
    attention kernel: no interpreted program, no separate soft-max launch, and the same values."""
    from cases import _np_decode_attention, decode_attention_ops, f32

    q, k, v = f32(1, (2, 8, 1, 64)), f32(2, (2, 2, 500, 64)), f32(3, (2, 2, 500, 64))
    hip.sync()
    hip.program_stats()
    out = decode_attention_ops(hip, hip.from_numpy(q), hip.from_numpy(k), hip.from_numpy(v), 4)
    got = hip.to_numpy(out)
    compiled, interpreted = hip.program_stats()
    assert (compiled, interpreted) == (1, 0)
    np.testing.assert_allclose(got, _np_decode_attention(q, k, v, 4), rtol=1e-4, atol=1e-5)
    # the same graph with 200 query positions per head: the one-pass prefill kernel
    q = f32(4, (2, 8, 200, 64))
    out = decode_attention_ops(hip, hip.from_numpy(q), hip.from_numpy(k), hip.from_numpy(v), 4)
    got = hip.to_numpy(out)
    assert hip.program_stats() == (1, 0)
    np.testing.assert_allclose(got, _np_decode_attention(q, k, v, 4), rtol=1e-4, atol=1e-5)
    # head_dim 128, a cache longer than the chunk
    q, k, v = f32(5, (1, 4, 100, 128)), f32(6, (1, 2, 150, 128)), f32(7, (1, 2, 150, 128))
    got = hip.to_numpy(decode_attention_ops(hip, hip.from_numpy(q), hip.from_numpy(k), hip.from_numpy(v), 2))
    assert hip.program_stats() == (1, 0)
    np.testing.assert_allclose(got, _np_decode_attention(q, k, v, 2), rtol=1e-4, atol=1e-5)


def test_norms_run_in_the_products_behind_them(hip):
    """The dense part of a decoder layer at decode time (hidden 2048, 4 rows): four skinny-product launches — o
    projection + residual add, gate / up / SiLU with the first norm in its loads, down projection + residual add,
    q / k / v with the second norm in their loads — and no launch for the norms or the adds (hidden 512
    and up, any multiple of 4).  With hidden 256 the products' kernels do not take the norms, which then run on their own:
    same values either way."""
    from catgrad_amd import _abi as A
    from cases import by_name

    classes = (A.K_GEMM_SKINNY, A.K_ELEMENTWISE, A.K_REDUCE)
    for name, fused in (("decoder_block_B4_H2048_F4096", True), ("decoder_block_B1_H1024_F3072", True), ("decoder_block_B4_H512_F4096", True),
                        ("decoder_block_B1_H576_F1536", True), ("decoder_block_B4_H256_F4096", False)):
        c = by_name(name)
        hip.sync()
        for cls in classes:
            hip.profile_enable(cls, 1)
            hip.profile_read(cls, True)
        got = c.run(hip)
        counts = tuple(hip.profile_read(cls, True)[0] for cls in classes)
        for cls in classes:
            hip.profile_enable(cls, 0)
        if fused:
            assert counts == (4, 0, 0), (name, counts)
        else:
            assert counts[0] >= 4 and counts[1] + counts[2] >= 2, (name, counts)
        for g, e in zip(got, c.expect()):
            np.testing.assert_allclose(g, e, rtol=1e-3, atol=4e-3)


def test_programs_absorbed_by_decode_time_products(hip):
    """gate and up projection of a decode step plus the SiLU program between them and the next product:
    one skinny-product launch and no element-wise launch; a pair the kernel does not take (8 rows) runs as
    a grouped product plus the compiled program and gives the same kind of result.  Likewise the residual
    adds around a product (eight sums per case): absorbed from 512 columns on, separate launches at 256."""
    from catgrad_amd import _abi as A
    from cases import by_name

    for name, launches in (("linear_gated_B4_K512_N4096", (1, 0)), ("linear_gated_B8_K512_N4096", (1, 1)),
                           ("linear_residual_B4_K512_N2048", (8, 0)), ("linear_residual_B4_K512_N512", (8, 0)),
                           ("linear_residual_B4_K512_N256", (8, 8))):
        c = by_name(name)
        hip.sync()
        for cls in (A.K_GEMM_SKINNY, A.K_ELEMENTWISE):
            hip.profile_enable(cls, 1)
            hip.profile_read(cls, True)
        got = c.run(hip)
        counts = tuple(hip.profile_read(cls, True)[0] for cls in (A.K_GEMM_SKINNY, A.K_ELEMENTWISE))
        for cls in (A.K_GEMM_SKINNY, A.K_ELEMENTWISE):
            hip.profile_enable(cls, 0)
        assert counts == launches, (name, counts)
        for g, e in zip(got, c.expect()):
            np.testing.assert_allclose(g, e, rtol=1e-3)


def test_rotary_embedding_and_cache_append_run_in_the_products_store(hip):
    """Two decode steps of an attention block (hidden 2048, 4 rows; hidden 1024, 1 row): the element-wise launches
    that remain are the two moves of the caches into buffers with room (first append) and the four read-backs of
    cache rows the case asks for; the rotary embedding of q and k and the writes of the new k / v rows cost none.
    With hidden 256 the products' kernel does not take the store and they run as a launch of their own per step."""
    from catgrad_amd import _abi as A
    from cases import by_name

    for name, ew in (("decode_qkv_rope_append_B4_K2048_kv8_rep4_T300_hd64_normed", 6),
                     ("decode_qkv_rope_append_B1_K1024_kv2_rep2_T256_hd128", 6),
                     ("decode_qkv_rope_append_B3_K512_kv4_rep2_T200_hd64", 6),
                     ("decode_qkv_rope_append_B1_K576_kv3_rep3_T200_hd64_normed", 6),
                     # q and k normed per head (the Qwen3 block): the norms run behind the products' store too (a small
                     # launch that is counted with the products, not with the element-wise ones), at any hidden size
                     ("decode_qkv_rope_append_B1_K1024_kv8_rep2_T300_hd128_qk_normed", 6),
                     ("decode_qkv_rope_append_B4_K1024_kv2_rep2_T200_hd64_qk", 6),
                     ("decode_qkv_rope_append_B2_K576_kv3_rep3_T131_hd64_qk_normed", 6),
                     ("decode_qkv_rope_append_B1_K2048_kv2_rep2_T100_hd128_qk_normed", 6),
                     # (head sizes other than 64 and 128: the attention's soft-max is a launch of its own per step)
                     ("decode_qkv_rope_append_B4_K2560_kv4_rep2_T77_hd96_qk_normed", 8),
                     ("decode_qkv_rope_append_B2_K1280_kv2_rep3_T63_hd80_qk", 8),
                     # (k and v of 48 columns are below what the products' kernels take)
                     ("decode_qkv_rope_append_B3_K4096_kv1_rep4_T40_hd48_qk_normed", None),
                     ("decode_qkv_rope_append_B3_K256_kv4_rep2_T200_hd64", None)):
        c = by_name(name)
        hip.sync()
        hip.profile_enable(A.K_ELEMENTWISE, 1)
        hip.profile_read(A.K_ELEMENTWISE, True)
        got = c.run(hip)
        count = hip.profile_read(A.K_ELEMENTWISE, True)[0]
        hip.profile_enable(A.K_ELEMENTWISE, 0)
        if ew is None:
            assert count > 6, (name, count)
        else:
            assert count == ew, (name, count)
        for g, e in zip(got, c.expect()):
            np.testing.assert_allclose(g, e, rtol=1e-3, atol=4e-3)


def test_backend_closes_with_writes_still_waiting():
    """Rows appended from a program and never read: the write is still waiting when the tensors and the
    backend go away."""
    from catgrad_amd import HipBackend

    be = HipBackend(0)
    cache = be.from_numpy(np.ones((2, 2, 8, 64), np.float32))
    for _ in range(2):
        new = be.neg(be.from_numpy(np.ones((2, 2, 1, 64), np.float32)).move())
        cache = be.concat(cache.move(), new.move(), 2)
    assert cache.shape == (2, 2, 10, 64)
    del cache, new
    be.close()


def test_one_backend_from_several_threads(hip):
    """Handles are `Send + Sync` in the reference (backend/mod.rs:124): several threads use one backend and
    shared input tensors at once — deferred programs, lazy products, appended rows, read-backs — and each gets
    the values it would get alone."""
    import threading

    rng = np.random.default_rng(11)
    w = (rng.standard_normal((4096, 512)) * 0.02).astype(np.float32)
    tw = hip.from_numpy(w)
    errors = []

    def work(seed):
        try:
            r = np.random.default_rng(seed)
            for it in range(12):
                x = np.abs(r.standard_normal((4, 1, 512)).astype(np.float32))
                tx = hip.from_numpy(x)
                y = hip.matmul(tx, hip.broadcast(hip.transpose(tw, 0, 1), (4, 512, 4096)))
                z = hip.exp(hip.neg(hip.mul(y, y)))
                cache = hip.from_numpy(np.zeros((2, 2, 300, 64), np.float32))
                rows = hip.add(hip.from_numpy(np.full((2, 2, 1, 64), float(seed), np.float32)),
                               hip.from_numpy(np.full((2, 2, 1, 64), float(it), np.float32)))
                cache = hip.concat(cache.move(), rows.move(), 2)
                got_z, got_c = hip.to_numpy(z), hip.to_numpy(cache)
                yy = x.astype(np.float64) @ w.astype(np.float64).T
                np.testing.assert_allclose(got_z, np.exp(-(yy * yy)), rtol=2e-3, atol=1e-6)
                assert got_c.shape == (2, 2, 301, 64) and np.all(got_c[:, :, 300] == seed + it) and not got_c[:, :, :300].any()
        except Exception as e:  # noqa: BLE001 - reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=work, args=(s,)) for s in range(1, 5)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_format_tensor(hip):
    s = hip.format_tensor(hip.from_numpy(np.array([[1.5, 2.0]], np.float32)))
    assert "f32[1,2]" in s and "1.5" in s


# ---- the narrow-operand products on the 16-bit and fp8 matrix instructions, many tiles deep -----------------
@pytest.mark.parametrize("dt", ["bf16", "f16", "fp8"])
def test_narrow_operand_products_deep_in_k_are_exact_on_integers(hip, dt):
    """Products that fill the device with 256 x 256 tiles run from operands narrowed in memory, through a loop whose
    steady state (whole tiles, loads dealt out between the matrix instructions) only starts three tiles deep in k.
    Small-integer operands make every partial sum an integer that f32 holds exactly, whatever the order of the additions,
    so the result must equal the rounding of the exact product bit for bit.  K = 1088 is 17 tiles of the 16-bit dtypes and
    8.5 of fp8 (a ragged last tile); 4000 x 4100 leaves ragged tile edges in both directions.  A second product against a
    0/1 selection matrix returns columns of the left operand unchanged: every position along k reaches its partner."""
    import cases_fp8
    import cases_half
    rng = np.random.default_rng(77)
    M, N, K = 4000, 4100, 1088
    if dt == "fp8":
        av = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        bv = (rng.integers(-1, 2, size=(N, K)) * (rng.random((N, K)) < 0.125)).astype(np.float32)
        up = lambda v: hip.ndarray_from_vec_fp8(cases_fp8.f8_encode(v), v.shape)
        rd = lambda t: cases_fp8.read(hip, t)
        rnd = cases_fp8.f8_round
    else:
        code = A.BF16 if dt == "bf16" else A.F16
        av = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
        bv = rng.integers(-8, 9, size=(N, K)).astype(np.float32)
        up = lambda v: cases_half.from_half(hip, code, cases_half.round_to(code, v))
        rd = lambda t: cases_half.as_f32(code, cases_half.read(hip, t))
        rnd = lambda x: cases_half.as_f32(code, cases_half.round_to(code, x))
    a, b = up(av), up(bv)
    got = rd(hip.matmul(a, hip.transpose(b, 0, 1)))
    exact = av.astype(np.float64) @ bv.astype(np.float64).T
    assert np.abs(exact).max() < 2 ** 24
    exp = rnd(exact.astype(np.float32))
    bad = np.argwhere(got != exp)
    assert bad.size == 0, f"{dt}: {len(bad)} mismatches, first {bad[:3].tolist()}"
    # selection: column n of the result is column sel[n] of the left operand
    sel = rng.integers(0, K, size=N)
    pv = np.zeros((N, K), dtype=np.float32)
    pv[np.arange(N), sel] = 1.0
    got = rd(hip.matmul(a, hip.transpose(up(pv), 0, 1)))
    assert np.array_equal(got, av[:, sel])


@pytest.mark.parametrize("dt", ["bf16", "f16", "fp8"])
def test_narrow_operand_products_carry_special_values(hip, dt):
    """NaN, infinities (16-bit dtypes) and the largest magnitudes through the narrowed-in-memory products: a NaN operand
    makes its whole row / column of the result NaN, inf x 0 is NaN, sums beyond the dtype's range come out as infinity
    (16-bit) or saturate at 448 (fp8), and everything else equals the rounding of the exact product (small integers)."""
    import cases_fp8
    import cases_half
    rng = np.random.default_rng(78)
    M, N, K = 4096, 4096, 256
    av = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
    bv = (rng.integers(-1, 2, size=(N, K)) * (rng.random((N, K)) < 0.125)).astype(np.float32)
    av[7, 3] = np.nan            # row 7 of the result is NaN
    bv[11, 200] = np.nan         # column 11 too
    big = 448.0 if dt == "fp8" else (3.0e38 if dt == "bf16" else 65504.0)
    av[100] = 0.0                # (nothing else in this row: sums that mix huge and small terms depend on the order of addition)
    av[100, :4] = big
    bv[:, :4] = 0.0
    bv[200, :4] = 1.0            # result[100, 200] = 4 x big exceeds the range
    bv[201, :4] = [1.0, -1.0, 0.0, 0.0]  # cancels exactly: stays finite
    if dt != "fp8":
        av[300, 5] = np.inf
        bv[400, 5] = 0.0         # inf x 0 = NaN at [300, 400]; elsewhere in row 300: +-inf or NaN by the signs of column 5
    if dt == "fp8":
        up = lambda v: hip.ndarray_from_vec_fp8(cases_fp8.f8_encode(v), v.shape)
        rd = lambda t: cases_fp8.read(hip, t)
        rnd = cases_fp8.f8_round
    else:
        code = A.BF16 if dt == "bf16" else A.F16
        up = lambda v: cases_half.from_half(hip, code, cases_half.round_to(code, v))
        rd = lambda t: cases_half.as_f32(code, cases_half.read(hip, t))
        rnd = lambda x: cases_half.as_f32(code, cases_half.round_to(code, x))
    got = rd(hip.matmul(up(av), hip.transpose(up(bv), 0, 1)))
    with np.errstate(invalid="ignore", over="ignore"):
        a_r, b_r = rnd(av).astype(np.float64), rnd(bv).astype(np.float64)   # (3.0e38 is not a bf16 value: what was uploaded)
        exact = a_r @ b_r.T
        exp = rnd(exact.astype(np.float32))
    same = (got == exp) | (np.isnan(got) & np.isnan(exp))
    bad = np.argwhere(~same)
    assert bad.size == 0, f"{dt}: {len(bad)} mismatches, first {bad[:3].tolist()}: got {got[tuple(bad[0])]} expected {exp[tuple(bad[0])]}"
    assert np.isnan(got[7]).all() and np.isnan(got[:, 11]).all()
    assert (np.isinf(got[100, 200]) if dt != "fp8" else got[100, 200] == 448.0) and np.isfinite(got[100, 201])
    if dt != "fp8":
        assert np.isnan(got[300, 400])


def _narrow_codec(hip, dt):
    import cases_fp8
    import cases_half
    if dt == "fp8":
        up = lambda v: hip.ndarray_from_vec_fp8(cases_fp8.f8_encode(v), v.shape)
        rd = lambda t: cases_fp8.read(hip, t)
        rnd = cases_fp8.f8_round
    else:
        code = A.BF16 if dt == "bf16" else A.F16
        up = lambda v: cases_half.from_half(hip, code, cases_half.round_to(code, v))
        rd = lambda t: cases_half.as_f32(code, cases_half.read(hip, t))
        rnd = lambda x: cases_half.as_f32(code, cases_half.round_to(code, x))
    return up, rd, rnd


def _small_integers(rng, dt, M, N, K):
    if dt == "fp8":
        av = rng.integers(-2, 3, size=(M, K)).astype(np.float32)
        bv = (rng.integers(-1, 2, size=(N, K)) * (rng.random((N, K)) < 0.125)).astype(np.float32)
    else:
        av = rng.integers(-8, 9, size=(M, K)).astype(np.float32)
        bv = rng.integers(-8, 9, size=(N, K)).astype(np.float32)
    return av, bv


@pytest.mark.parametrize("dt", ["bf16", "f16", "fp8"])
@pytest.mark.parametrize("shape", ["ragged_edges", "partial_last_round"])
def test_narrow_operand_products_through_the_lds_ring_are_exact_on_integers(hip, hip_words_only, dt, shape):
    """Rows of k that are whole turns of the four-stage ring (multiples of 128 values of the 16-bit dtypes, of 256 of fp8)
    take the kernel whose loads go straight into LDS and whose workgroups walk the tiles: one per compute unit, so 17 x 16
    tiles end with a round in which few workgroups have a tile left, and 32 x 33 tiles take four full rounds and a partial
    one.  The 16-bit dtypes round the result in that kernel's store (two columns per lane, exchanged between neighbours);
    with 32-bit storage (the second backend) the same kernel stores f32 words and the rounding pass follows.  Small
    integers make the exact product the only right answer (see the test above); 4000 x 4100 leaves ragged tiles at both
    edges, which take the guarded store; a sliced left operand has a row pitch of twice its width."""
    rng = np.random.default_rng(79)
    M, N, K = (4000, 4100, 1280) if shape == "ragged_edges" else (8192, 8448, 256)
    av, bv = _small_integers(rng, dt, M, N, K)
    exp32 = av @ bv.T                                   # (sgemm on small integers: every partial sum is exact)
    assert np.abs(exp32).max() < 2 ** 24
    for be in (hip, hip_words_only):
        print(f"dt={dt} shape={shape} storage={'words' if be is hip_words_only else 'narrow'}", flush=True)
        up, rd, rnd = _narrow_codec(be, dt)
        exp = rnd(exp32)
        a, b = up(av), up(bv)
        got = rd(be.matmul(a, be.transpose(b, 0, 1)))
        bad = np.argwhere(got != exp)
        assert bad.size == 0, f"{dt}: {len(bad)} mismatches, first {bad[:3].tolist()}"
        if shape == "ragged_edges":
            # the left operand as the right half of a tensor twice as wide
            wide = up(np.concatenate([np.zeros_like(av), av], axis=1))
            got = rd(be.matmul(be.slice(wide, 1, K, K), be.transpose(b, 0, 1)))
            assert np.array_equal(got, exp)
        del a, b, got


@pytest.mark.parametrize("n", [2, 63, 64, 65, 1023, 1024, 1025, 5000])
def test_small_uploads_and_read_backs_on_both_paths(hip, n):
    """Up to 64 words go up as the arguments of a small kernel and up to 1024 come back through pinned memory that the host
    polls; beyond that, and with CG_FAST_READBACK=0, the runtime's staged copies and the stream's own wait do it.  Both
    paths, at the limits, f32 and u32, a view that has to be gathered first, and a read-back right behind a long launch."""
    from backends import backend_with_env

    rng = np.random.default_rng(n)
    xv = rng.standard_normal(n).astype(np.float32)
    iv = rng.integers(0, 2 ** 32, size=n, dtype=np.uint32)
    big = rng.standard_normal((2048, 2048)).astype(np.float32)
    slow = backend_with_env(CG_FAST_READBACK="0")
    try:
        for be in (hip, slow):
            assert np.array_equal(be.to_numpy(be.from_numpy(xv)), xv)
            assert np.array_equal(be.to_numpy(be.from_numpy(iv)), iv)
            x2 = be.from_numpy(np.stack([xv, -xv]))
            assert np.array_equal(be.to_numpy(be.slice(be.transpose(x2, 0, 1), 1, 1, 1)), -xv.reshape(n, 1))
            # behind a launch of a few hundred microseconds: the words must be those of the finished product
            b = be.from_numpy(big)
            p = be.matmul(b, b)
            got = be.to_numpy(be.slice(be.reshape(p, (2048 * 2048,)), 0, 7, min(n, 1024)))
            ref = (big.astype(np.float64) @ big.astype(np.float64)).reshape(-1)[7:7 + min(n, 1024)]
            np.testing.assert_allclose(got, ref, rtol=1e-3, atol=1e-2)
    finally:
        slow.close()


# ---- full-size checks through size-independent properties -----------------------------------
def test_microbench_shapes_properties(hip):
    """Config-2 shapes: linearity / invariants instead of a CPU recomputation."""
    rng = np.random.default_rng(0)
    n = 8192
    row = rng.standard_normal((1, n)).astype(np.float32)
    big = hip.broadcast(hip.from_numpy(row), (4096, n))
    # sum over the last axis of a row-broadcast tensor: every row gives the same value
    s = hip.to_numpy(hip.sum(big))
    ref = np.float64(row.astype(np.float64).sum())
    assert s.shape == (4096, 1)
    assert np.all(s == s[0])
    assert abs(float(s[0, 0]) - ref) <= 1e-3 * np.abs(row).astype(np.float64).sum()
    m = hip.to_numpy(hip.max(big))
    assert np.all(m == row.max())
    am = hip.to_numpy(hip.argmax(big))
    assert np.all(am == np.uint32(n - 1 - np.argmax(row[0, ::-1])))
    # exp(a + b) == exp(a) * exp(b) on [8192, 8192]
    a = hip.from_numpy((rng.standard_normal((n, n)) * 0.5).astype(np.float32))
    b = hip.from_numpy((rng.standard_normal((n, n)) * 0.5).astype(np.float32))
    lhs = hip.exp(hip.add(a, b))
    rhs = hip.mul(hip.exp(a), hip.exp(b))
    d = hip.to_numpy(hip.max(hip.reshape(hip.div(hip.sub(lhs.clone(), rhs), lhs), (1, n * n))))
    assert float(d[0, 0]) < 1e-5
    # bmm [16,1024,1024]: (A B) 1 == A (B 1)
    a_np = rng.standard_normal((16, 1024, 1024)).astype(np.float32)
    b_np = rng.standard_normal((16, 1024, 1024)).astype(np.float32)
    A_, B_ = hip.from_numpy(a_np), hip.from_numpy(b_np)
    ones = hip.broadcast(hip.from_numpy(np.float32(1).reshape(())), (16, 1024, 1))
    prod = hip.matmul(A_, B_)
    left = hip.to_numpy(hip.matmul(prod, ones))
    right = hip.to_numpy(hip.matmul(A_, hip.matmul(B_, ones)))
    # both sides against float64, 1e-3 of the scale of the terms summed (sum_k |a| * |sum_n b|, resp. sum_n |(ab)|)
    a64, b64 = a_np.astype(np.float64), b_np.astype(np.float64)
    b1 = b64.sum(-1, keepdims=True)
    exact = a64 @ b1
    scale_r = np.abs(a64) @ np.abs(b1)
    assert (np.abs(right - exact) <= 1e-3 * scale_r).all()
    assert (np.abs(left - exact) <= 1e-3 * scale_r).all()
    # sampled rows of the product itself in float64: 1e-3 of sum_k |a| |b|
    full = hip.to_numpy(prod)
    for bi, r in ((0, 0), (5, 1023), (15, 517), (9, 64)):
        ex = a64[bi, r] @ b64[bi]
        sc = np.abs(a64[bi, r]) @ np.abs(b64[bi])
        assert (np.abs(full[bi, r] - ex) <= 1e-3 * sc).all()


@pytest.mark.parametrize("shape", [(1500, 8192), (2, 1100, 4096), (8192, 8192)])
def test_reductions_over_a_strided_axis_with_many_outputs(hip, shape):
    """`sum` / `max` / `argmax` over the last axis of a transposed view with 8192 outputs and a long reduced axis (the
    extents of the micro-benchmark's sum over axis 0, a ragged length, a batched one): the shapes that take the one-launch
    column kernel.  sum within 1e-3 of sum |x| against float64, max exact, argmax bit-exact (planted ties: the last wins)."""
    rng = np.random.default_rng(77 + len(shape))
    x = rng.standard_normal(shape).astype(np.float32)
    n = shape[-2]
    x[..., 5, 64] = x[..., n - 3, 64] = np.float32(9.5)      # equal maxima down a column: the last one wins
    x[..., :, 65] = np.float32(-1.25)                         # a column of equal values: index n - 1
    x[..., 700, 66] = np.float32(np.nan)                      # +NaN: greatest for argmax, ignored by max, NaN sum
    t = hip.transpose(hip.from_numpy(x), len(shape) - 2, len(shape) - 1)
    xt = np.swapaxes(x, -1, -2)
    x64 = xt.astype(np.float64)
    s = hip.to_numpy(hip.sum(t.clone()))[..., 0]
    ok = ~np.isnan(x64.sum(-1))
    assert s.shape == xt.shape[:-1]
    assert np.all(np.abs(s[ok] - x64.sum(-1)[ok]) <= 1e-3 * np.abs(x64).sum(-1)[ok])
    assert np.isnan(s[~ok]).all() and (~ok).sum() == int(np.prod(shape[:-2]))
    m = hip.to_numpy(hip.max(t.clone()))[..., 0]
    np.testing.assert_array_equal(m, np.fmax.reduce(xt, axis=-1))
    am = hip.to_numpy(hip.argmax(t))[..., 0]
    i32 = np.ascontiguousarray(xt).view(np.int32).astype(np.int64)
    key = np.where(i32 < 0, -(i32 & 0x7FFFFFFF) - 1, i32)    # total_cmp order of the bit patterns (ndarray.rs:670-681)
    ref_am = (n - 1 - np.argmax(key[..., ::-1], axis=-1)).astype(np.uint32)
    np.testing.assert_array_equal(am, ref_am)
    assert (am[..., 64] == n - 3).all() and (am[..., 65] == n - 1).all() and (am[..., 66] == 700).all()


def test_microbench_dense_reductions(hip):
    """Config-2 reductions on a DENSE random f32[4096, 8192] (the extent and kernel path the micro-benchmark times):
    sum within 1e-3 of sum |x| against float64, max exact, argmax bit-exact with the last of equal maxima (planted ties,
    a row of equal values, a +NaN, -0.0 against +0.0)."""
    rng = np.random.default_rng(42)
    x = rng.standard_normal((4096, 8192)).astype(np.float32)
    x[7, 100] = x[7, 8000] = np.float32(9.5)        # equal maxima: the last one wins
    x[8, :] = np.float32(-1.25)                      # every element equal: index n - 1
    x[9, 4321] = np.float32(np.nan)                  # +NaN is greatest in total order for argmax, ignored by max
    x[10, :] = np.float32(-0.0)
    x[10, 17] = np.float32(0.0)                      # +0.0 beats -0.0 in total order
    t = hip.from_numpy(x)
    s = hip.to_numpy(hip.sum(t.clone()))
    x64 = x.astype(np.float64)
    ok = np.ones(4096, bool)
    ok[9] = False                                    # the NaN row sums to NaN
    assert s.shape == (4096, 1)
    assert np.all(np.abs(s[ok, 0] - x64[ok].sum(-1)) <= 1e-3 * np.abs(x64[ok]).sum(-1))
    assert np.isnan(s[9, 0])
    m = hip.to_numpy(hip.max(t.clone()))
    ref_max = np.fmax.reduce(x, axis=-1)             # NaN ignored, as f32::max does (ndarray.rs:656-668)
    np.testing.assert_array_equal(m[:, 0], ref_max)
    am = hip.to_numpy(hip.argmax(t))[:, 0]
    i32 = x.view(np.int32).astype(np.int64)
    key = np.where(i32 < 0, -(i32 & 0x7FFFFFFF) - 1, i32)   # total_cmp order of the bit patterns (ndarray.rs:670-681)
    ref_am = (8192 - 1 - np.argmax(key[:, ::-1], axis=-1)).astype(np.uint32)
    np.testing.assert_array_equal(am, ref_am)
    assert am[7] == 8000 and am[8] == 8191 and am[9] == 4321 and am[10] == 17

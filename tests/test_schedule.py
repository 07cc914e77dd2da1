"""The host driver's second evaluation mode: a model run recorded as a term and evaluated in the layers of the
reference's evaluator (catgrad/src/abstract_interpreter/eval.rs:38-66, catgrad/src/ssa/mod.rs:24-76) with its
move / clone value map, against the order in which the graph builder issues the operations.  Operations are pure, so
on one backend the schedules must agree bit for bit (CPU oracle); on the GPU the fused paths that recognise patterns
in the order of calls must give the same values, and stay in use, under either order.  Also the two known answers of
catgrad/tests/test_if.rs for `If` (`handle_if`, interpreter.rs:86-107)."""
import numpy as np
import pytest

import np_models
from catgrad_amd import _abi as A
from catgrad_amd.runner import LlmConfig, Session, random_params
from model_cases import TINY, params_of, prompt_of
from oracle_loader import ORACLE_LIB, oracle_library


@pytest.mark.parametrize("name", list(TINY))
def test_oracle_schedules_agree_bit_for_bit(name):
    oracle_library()
    cfg = TINY[name]
    params = params_of(cfg, seed=11, scale=4.0)
    prompt = prompt_of(cfg, 3, 10, seed=12)
    outs = []
    for schedule in (0, 1, 2):
        s = Session(ORACLE_LIB)
        s.set_schedule(schedule)
        s.load_model(cfg, params=params.items())
        gen, st = s.generate(prompt, steps=6, max_positions=32)
        toks, logits = s.forward(prompt, max_positions=32)
        outs.append((gen, toks, logits, st["prefill_calls"], st["decode_calls"]))
        s.close()
    for gen, toks, logits, pc, dc in outs[1:]:
        np.testing.assert_array_equal(gen, outs[0][0])
        np.testing.assert_array_equal(toks, outs[0][1])
        np.testing.assert_array_equal(logits, outs[0][2])
        assert (pc, dc) == outs[0][3:]          # the same backend calls, in another order
    # and the values are the model's: float64 numpy on the same weights
    l64 = np_models.llm_logits(cfg, params, prompt)
    assert np.abs(outs[1][2] - l64).max() <= 1e-3 * np.abs(l64).max()


@pytest.mark.parametrize("schedule", [0, 1, 2])
def test_if_known_answers_oracle(schedule):
    """test_if.rs: cond(c, then: x + x, else: x, [x]) with x = 5: c = 1 gives 10, c = 0 gives 5."""
    oracle_library()
    s = Session(ORACLE_LIB)
    s.set_schedule(schedule)
    assert s.cond_kat(5.0, 1.0) == 10.0
    assert s.cond_kat(5.0, 0.0) == 5.0
    assert s.cond_kat(5.0, float("nan")) == 5.0      # to_bool: NaN > 0 is false (ndarray.rs:140-149)
    assert s.cond_kat(-2.5, 0.25) == -5.0
    s.close()


@pytest.mark.gpu
@pytest.mark.parametrize("schedule", [0, 1, 2])
def test_if_known_answers_hip(schedule):
    s = Session()
    s.set_schedule(schedule)
    assert s.cond_kat(5.0, 1.0) == 10.0
    assert s.cond_kat(5.0, 0.0) == 5.0
    assert s.cond_kat(5.0, float("nan")) == 5.0
    s.close()


def _decode_shapes():
    # tiny models, and one with the widths at which the decode-time products absorb norms, residual adds and the
    # SiLU pair (hidden a multiple of 1024, at most 4 rows)
    yield "tiny_llama", TINY["tiny_llama"], 4.0, 3
    yield "tiny_qwen3", TINY["tiny_qwen3"], 4.0, 3
    yield "llama_h1024", LlmConfig("llama", 1024, 3, 16, 4, 2048, 1000, rope_theta=500000.0, tie_word_embeddings=True), 1.0, 4
    yield "qwen3_h1024", LlmConfig("qwen3", 1024, 2, 8, 4, 3072, 1200, head_dim=128, rms_norm_eps=1e-6, rope_theta=1000000.0,
                                   tie_word_embeddings=True), 1.0, 1


@pytest.mark.gpu
@pytest.mark.parametrize("name,cfg,scale,B", list(_decode_shapes()), ids=[c[0] for c in _decode_shapes()])
def test_hip_under_the_reference_schedule(name, cfg, scale, B):
    oracle_library()
    params = params_of(cfg, seed=21, scale=scale)
    prompt = prompt_of(cfg, B, 12, seed=22)
    steps = 6
    cpu = Session(ORACLE_LIB)
    cpu.load_model(cfg, params=params.items())
    g_c, _, l_c = cpu.generate(prompt, steps=steps, max_positions=32, want_logits=True)
    cpu.close()
    seq = np.concatenate([prompt, g_c[:-1].T], axis=1)
    l64 = np_models.llm_logits(cfg, params, seq, positions=range(11, 12 + steps))
    srt = np.sort(l64, -1)
    gaps = (srt[..., -1] - srt[..., -2]).T
    scale_l = float(np.abs(l_c).max())
    stats, launches = {}, {}
    for schedule in (0, 1, 2):
        hip = Session()
        hip.set_schedule(schedule)
        hip.load_model(cfg, params=params.items())
        hip.program_stats()
        hip.profile_enable(A.K_ELEMENTWISE, 1)
        hip.profile_read(A.K_ELEMENTWISE, True)
        g_h, st, l_h = hip.generate(prompt, steps=steps, max_positions=32, want_logits=True)
        stats[schedule] = hip.program_stats()
        launches[schedule] = hip.profile_read(A.K_ELEMENTWISE, True)[0]
        hip.close()
        err = float(np.abs(l_h - l_c).max())
        print(f"{name} schedule {schedule}: max |dlogit| {err:.3e} (scale {scale_l:.3e}); fused programs compiled / "
              f"interpreted {stats[schedule]}; mismatches {int((g_h != g_c).sum())}", flush=True)
        assert err <= 1e-3 * scale_l
        for b in range(B):
            d = np.flatnonzero(g_h[:, b] != g_c[:, b])
            assert d.size == 0 or gaps[d[0], b] <= 2 * max(err, 1e-6 * scale_l)
    # the fused paths are found under either order: no more launches of fused programs than in the builder's order
    # (each absorbed program is one launch fewer), and nothing new falls to the interpreter kernels
    for schedule in (1, 2):
        assert stats[schedule][1] <= stats[0][1]
        assert stats[schedule][0] <= stats[0][0] * 1.02 + 2
        # nor more element-wise launches: the rotary embedding and the cache rows still go into the q / k / v store
        assert launches[schedule] <= launches[0] + 2, (launches, name)
    print(f"{name}: element-wise launches per schedule {launches}", flush=True)

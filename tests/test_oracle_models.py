"""Pins the host driver (interpreter mirror + model graphs) running on the CPU oracle
against independent float64 numpy statements of the same mathematics."""
import numpy as np
import pytest

import np_models
from catgrad_amd.runner import Session
from model_cases import TINY, load_mlp, mlp_case, params_of, prompt_of
from oracle_loader import ORACLE_LIB, oracle_library


@pytest.fixture(scope="module")
def session():
    oracle_library()
    return Session(ORACLE_LIB)


@pytest.mark.parametrize("name", list(TINY))
def test_logits_match_float64_model(session, name):
    cfg = TINY[name]
    params = params_of(cfg, seed=3, scale=4.0)
    session.load_model(cfg, params=params.items())
    prompt = prompt_of(cfg, 2, 9)
    toks, logits = session.forward(prompt, max_positions=16)
    ref = np_models.llm_logits(cfg, params, prompt)
    scale = np.abs(ref).max()
    assert np.abs(logits - ref).max() <= 1e-3 * scale  # matmul/reduction contract
    np.testing.assert_array_equal(toks, ref.argmax(-1).astype(np.uint32))


@pytest.mark.parametrize("name", list(TINY))
def test_greedy_decode_with_kv_cache_matches_full_recomputation(session, name):
    cfg = TINY[name]
    params = params_of(cfg, seed=5, scale=4.0)
    session.load_model(cfg, params=params.items())
    prompt = prompt_of(cfg, 3, 6, seed=7)
    toks, stats = session.generate(prompt, steps=8, max_positions=14)
    ref, gaps = np_models.greedy(cfg, params, prompt, 8)
    # a flip is only a defect if the float64 top1-top2 gap exceeds the 1e-3 envelope
    decisive = gaps > 1e-3 * 10.0
    agree = toks == ref
    first_bad = np.argwhere(~agree)
    if first_bad.size:
        step, b = first_bad[0]
        assert not decisive[step, b], f"token flip at step {step}, row {b} with gap {gaps[step, b]:.3e}"
    else:
        assert agree.all()
    assert stats["prefill_calls"] > 0 and stats["decode_calls"] > 0


def test_config1_mlp(session):
    case = mlp_case(0)
    load_mlp(session, case)
    y = session.mlp(case[0], 512, 10)
    ref = np_models.mlp(*case)
    assert y.shape == (1, 64, 10)
    np.testing.assert_allclose(y[0], ref, rtol=1e-3, atol=1e-5)

"""The LLM helper compositions and the interpreter's side doors, through the host driver on any backend:
  * known answers of catgrad-llm/src/helpers_tests.rs (repeat_kv, repeat_interleave, cumsum) from
    tests/golden/helper_kats.json, under the three evaluation orders;
  * `Probe` (catgrad/src/interpreter/tensor_op.rs:121-136): silent unless CATGRAD_PROBE is set, then
    "[probe:label] <format_tensor>", no result either way;
  * a Definition (`nn::Sigmoid.call`, catgrad/src/interpreter/interpreter.rs:61-74) as one operation of the recorded
    term: the config-1 MLP gives the same bits under every schedule;
  * an `If` whose branches disagree in type is rejected while the term is recorded."""
import json
import os

import numpy as np
import pytest

from catgrad_amd.runner import Session
from oracle_loader import ORACLE_LIB, oracle_library

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "helper_kats.json")) as f:
    HELPER_KATS = json.load(f)["cases"]


def _session(on_gpu, schedule):
    if on_gpu:
        s = Session()
    else:
        oracle_library()
        s = Session(ORACLE_LIB)
    s.set_schedule(schedule)
    return s


def _helper_kats(on_gpu, schedule):
    s = _session(on_gpu, schedule)
    for case in HELPER_KATS:
        x = np.array(case["input"]["data"], dtype=np.float32).reshape(case["input"]["shape"])
        got = s.helper(case["helper"], x, case["a0"], case["a1"])
        exp = np.array(case["expect"]["data"], dtype=np.float32).reshape(case["expect"]["shape"])
        assert got.shape == exp.shape, case["name"]
        np.testing.assert_array_equal(got, exp, err_msg=case["name"])  # small integers: exact in any order
    # beyond the literals: the closed forms on random data (repeat = np.repeat, cumsum = np.cumsum in float64)
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 3, 5, 8), dtype=np.float32)
    np.testing.assert_array_equal(s.helper("repeat_kv", x, 4), np.repeat(x, 4, axis=1))
    np.testing.assert_array_equal(s.helper("repeat_interleave", x, 2, 3), np.repeat(x, 3, axis=2))
    c = s.helper("cumsum", x)
    ref = np.cumsum(x.astype(np.float64), axis=-1)
    assert np.abs(c - ref).max() <= 1e-3 * np.abs(x).sum(-1).max()
    s.close()


@pytest.mark.parametrize("schedule", [0, 1, 2])
def test_helper_known_answers_oracle(schedule):
    _helper_kats(False, schedule)


@pytest.mark.gpu
@pytest.mark.parametrize("schedule", [0, 1, 2])
def test_helper_known_answers_hip(schedule):
    _helper_kats(True, schedule)


def _probe(on_gpu, schedule, capfd, monkeypatch):
    x = np.array([[1.5, -2.0], [3.0, 4.25]], dtype=np.float32)
    s = _session(on_gpu, schedule)
    monkeypatch.delenv("CATGRAD_PROBE", raising=False)
    capfd.readouterr()
    y = s.helper("probe", x, label="quiet")
    assert "[probe:" not in capfd.readouterr().out            # no output, and the value passes through untouched
    np.testing.assert_array_equal(y, x)
    monkeypatch.setenv("CATGRAD_PROBE", "1")
    y = s.helper("probe", x, label="after_norm")
    out = capfd.readouterr().out
    np.testing.assert_array_equal(y, x)
    lines = [l for l in out.splitlines() if l.startswith("[probe:")]
    assert len(lines) == 1
    assert lines[0].startswith("[probe:after_norm] f32[2,2] [1.5, -2, 3, 4.25]"), lines[0]
    s.close()


@pytest.mark.parametrize("schedule", [0, 1])
def test_probe_oracle(schedule, capfd, monkeypatch):
    _probe(False, schedule, capfd, monkeypatch)


@pytest.mark.gpu
@pytest.mark.parametrize("schedule", [0, 1])
def test_probe_hip(schedule, capfd, monkeypatch):
    _probe(True, schedule, capfd, monkeypatch)


def _mlp_under_schedules(on_gpu):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((64, 256), dtype=np.float32)
    w1 = rng.standard_normal((512, 256), dtype=np.float32) * np.float32(0.02)
    w2 = rng.standard_normal((10, 512), dtype=np.float32) * np.float32(0.02)
    outs = []
    for schedule in (0, 1, 2):
        s = _session(on_gpu, schedule)
        s.set_param("mlp.l1.weight", w1)
        s.set_param("mlp.l1.bias", np.zeros(512, np.float32))
        s.set_param("mlp.l2.weight", w2)
        s.set_param("mlp.l2.bias", np.zeros(10, np.float32))
        outs.append(s.mlp(x, 512, 10))
        s.close()
    h = 1.0 / (1.0 + np.exp(-(x.astype(np.float64) @ w1.T.astype(np.float64))))
    ref = h @ w2.T.astype(np.float64)
    for o in outs:
        assert np.abs(o[0] - ref).max() <= 1e-3 * np.abs(ref).max()
    return outs


def test_definition_is_one_operation_oracle():
    outs = _mlp_under_schedules(False)
    np.testing.assert_array_equal(outs[1], outs[0])   # pure operations: the order cannot change a bit on one backend
    np.testing.assert_array_equal(outs[2], outs[0])


@pytest.mark.gpu
def test_definition_is_one_operation_hip():
    _mlp_under_schedules(True)


@pytest.mark.parametrize("schedule", [1, 2])
def test_if_branches_must_agree_in_type(schedule):
    s = _session(False, schedule)
    with pytest.raises(RuntimeError, match="branches of If disagree"):
        s.cond_mismatch()
    s.close()

"""Pins the CPU oracle against what the mathematics fixes: numpy closed forms for
integer / shape / index ops (bit-exact), float64 evaluation for f32 math, brute-force
rules for argmax / max / topk / cast special cases."""
import numpy as np
import pytest

from cases import CASES, assert_close


@pytest.mark.parametrize("case", [c for c in CASES if c.expect is not None], ids=lambda c: c.name)
def test_oracle_matches_closed_form(oracle, case):
    got = case.run(oracle)
    exp = case.expect()
    scales = case.scale() if case.scale else [None] * len(exp)
    assert len(got) == len(exp)
    for i, (g, e, s) in enumerate(zip(got, exp, scales)):
        assert_close(case.kind, g, e, s, f"{case.name}[{i}]")

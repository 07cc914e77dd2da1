"""Pins the CPU oracle against every known answer the reference's own tests hold for
the Backend path (transcribed in tests/golden/backend_kats.json)."""
import pytest

from catgrad_amd.backend import BackendPanic
from kat_runner import KATS, apply, check_case


@pytest.mark.parametrize("case", KATS["cases"], ids=lambda c: c["name"])
def test_kat(oracle, case):
    check_case(oracle, case)


@pytest.mark.parametrize("case", KATS["errors"], ids=lambda c: c["name"])
def test_error(oracle, case):
    with pytest.raises(BackendPanic) as e:
        apply(oracle, case)
    if "message" in case:
        assert case["message"] in str(e.value)

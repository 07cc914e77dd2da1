"""The C-ABI libraries load and export every symbol include/catgrad_hip.h declares
(no compute calls: this runs without a GPU)."""
import ctypes
import os
import re

import pytest

from catgrad_amd import _abi
from catgrad_amd.backend import HIP_LIBRARY

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "catgrad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cg_[a-z_0-9]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert declared_symbols() == sorted(_abi.SIGNATURES)


@pytest.mark.parametrize("which", ["hip", "oracle"])
def test_library_exports_every_symbol(which):
    if which == "hip":
        assert os.path.exists(HIP_LIBRARY), "build the HIP library first (__graft_entry__.build())"
        lib = ctypes.CDLL(HIP_LIBRARY, mode=ctypes.RTLD_LOCAL)
    else:
        from oracle_loader import oracle_library

        lib = oracle_library()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{which} library lacks {name}"


def test_hip_backend_refuses_to_run_without_a_gpu_or_library():
    """The product has no CPU fallback: creating a backend without a device is an error."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from catgrad_amd import BackendPanic, HipBackend

    with pytest.raises((BackendPanic, RuntimeError)):
        HipBackend(0)

"""Loads the CPU oracle (oracle/liboracle.so) for use as the checker in tests."""
import os
import subprocess

from catgrad_amd import _abi
from catgrad_amd.backend import Backend

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_DIR = os.path.join(ROOT, "oracle")
ORACLE_LIB = os.path.join(ORACLE_DIR, "liboracle.so")

_lib = None


def oracle_library():
    global _lib
    if _lib is None:
        if not os.path.exists(ORACLE_LIB):
            subprocess.check_call(["make", "-C", ORACLE_DIR])
        _lib = _abi.bind(ORACLE_LIB)
    return _lib


def oracle_backend() -> Backend:
    return Backend(oracle_library())

"""Weight ingest: safetensors files -> backend parameters (catgrad-llm/src/utils/mod.rs:321-449).

The files are written with the `safetensors` package itself, so the header reader of the host
driver is checked against the real format (metadata block, padding, dtype names).  bfloat16
values must arrive as exactly `bits << 16` (utils/mod.rs:158-168); I64 tensors are skipped;
any other dtype is an error; byte ranges are validated."""
import json
import os
import struct

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

from catgrad_amd.runner import Session, random_params
from model_cases import TINY, params_of, prompt_of
from oracle_loader import ORACLE_LIB, oracle_library


def bf16_round(w):
    """float32 -> nearest-even bfloat16 -> float32 (what a bf16 checkpoint holds)."""
    return torch.from_numpy(np.ascontiguousarray(w)).to(torch.bfloat16)


def write_checkpoint(path, cfg, params, bf16_names=lambda n: n.endswith("proj.weight")):
    tensors, expect = {}, {}
    for name, w in params.items():
        if bf16_names(name):
            t = bf16_round(w)
            tensors[name] = t
            expect[name] = t.to(torch.float32).numpy()
        else:
            tensors[name] = torch.from_numpy(np.ascontiguousarray(w))
            expect[name] = w
    tensors["bn.num_batches_tracked"] = torch.tensor([7], dtype=torch.int64)  # skipped by the loader
    save_file(tensors, path, metadata={"format": "pt", "note": 'quotes " and \\ backslashes'})
    return expect


def run_case(session, tmp_path, name="tiny_llama"):
    cfg = TINY[name]
    params = params_of(cfg, seed=21, scale=4.0)
    path = os.path.join(tmp_path, "model.safetensors")
    expect = write_checkpoint(path, cfg, params)
    st = session.load_safetensors(path, cfg)
    assert st["tensors"] == len(params)
    assert st["params"] == sum(w.size for w in params.values())
    prompt = prompt_of(cfg, 2, 9, seed=22)
    _, logits_file = session.forward(prompt, max_positions=16)
    session.load_model(cfg, params=expect.items())
    _, logits_mem = session.forward(prompt, max_positions=16)
    session.clear_params()
    np.testing.assert_array_equal(logits_file, logits_mem)


def test_oracle_loads_safetensors(tmp_path):
    oracle_library()
    s = Session(ORACLE_LIB)
    run_case(s, tmp_path)
    s.close()


def test_two_files_and_sharded_names(tmp_path):
    oracle_library()
    s = Session(ORACLE_LIB)
    cfg = TINY["tiny_qwen3"]
    params = params_of(cfg, seed=3)
    names = sorted(params)
    a, b = os.path.join(tmp_path, "a.safetensors"), os.path.join(tmp_path, "b.safetensors")
    save_file({n: torch.from_numpy(np.ascontiguousarray(params[n])) for n in names[::2]}, a)
    save_file({n: bf16_round(params[n]) for n in names[1::2]}, b)
    st = s.load_safetensors([a, b], cfg)
    assert st["tensors"] == len(names)
    assert st["bytes"] == sum(params[n].size * (4 if i % 2 == 0 else 2) for i, n in enumerate(names))
    s.close()


def _raw_file(path, header: dict, data: bytes):
    h = json.dumps(header).encode()
    with open(path, "wb") as f:
        f.write(struct.pack("<Q", len(h)) + h + data)


def test_rejects_bad_files(tmp_path):
    oracle_library()
    s = Session(ORACLE_LIB)
    p = os.path.join(tmp_path, "bad.safetensors")
    save_file({"w": torch.zeros(4, dtype=torch.float16)}, p)
    with pytest.raises(RuntimeError, match="UnsupportedDtype\\(F16\\)"):
        s.load_safetensors(p)
    _raw_file(p, {"w": {"dtype": "F32", "shape": [3], "data_offsets": [0, 16]}}, b"\0" * 16)
    with pytest.raises(RuntimeError, match="does not match its shape"):
        s.load_safetensors(p)
    _raw_file(p, {"w": {"dtype": "F32", "shape": [4], "data_offsets": [0, 16]}}, b"\0" * 12)
    with pytest.raises(RuntimeError, match="does not match its shape"):
        s.load_safetensors(p)
    with open(p, "wb") as f:
        f.write(struct.pack("<Q", 1 << 40) + b"{}")
    with pytest.raises(RuntimeError, match="header length exceeds"):
        s.load_safetensors(p)
    with open(p, "wb") as f:
        f.write(b"\1\2\3")
    with pytest.raises(RuntimeError, match="not a safetensors file"):
        s.load_safetensors(p)
    with pytest.raises(RuntimeError, match="cannot open"):
        s.load_safetensors(os.path.join(tmp_path, "missing.safetensors"))
    _raw_file(p, {"w": {"dtype": "F32", "shape": [2]}}, b"\0" * 8)
    with pytest.raises(RuntimeError, match="incomplete tensor entry"):
        s.load_safetensors(p)
    s.close()


def test_bf16_widening_is_a_shift(oracle):
    bits = np.array([0x0000, 0x8000, 0x3F80, 0xBF80, 0x7F80, 0xFF80, 0x7FC0, 0x0001, 0x7F7F, 0x4049], np.uint16)
    got = oracle.to_numpy(oracle.from_bf16_bits(bits, (2, 5)))
    exp = (bits.astype(np.uint32) << 16).view(np.float32).reshape(2, 5)
    np.testing.assert_array_equal(got.view(np.uint32), exp.view(np.uint32))


@pytest.mark.gpu
def test_hip_loads_safetensors(tmp_path):
    s = Session()
    for name in ("tiny_llama", "tiny_qwen3"):
        run_case(s, tmp_path, name)
    s.close()


@pytest.mark.gpu
@pytest.mark.parametrize("n", [1, 2, 7, 8, 9, 4096, 1000003])
def test_hip_bf16_widening_matches_shift(hip, n):
    bits = np.random.default_rng(n).integers(0, 1 << 16, size=n, dtype=np.uint16)
    got = hip.to_numpy(hip.from_bf16_bits(bits, (n,)))
    np.testing.assert_array_equal(got.view(np.uint32), bits.astype(np.uint32) << 16)


@pytest.mark.gpu
def test_hip_large_upload_is_staged_in_chunks(hip):
    """An upload larger than the two 16 MiB pinned staging buffers together, followed at once by
    a second one: chunking and buffer reuse must not mix the two."""
    rng = np.random.default_rng(5)
    a = rng.standard_normal((3, 5_000_011)).astype(np.float32)   # 60 MB, ragged against the chunk size
    b = rng.integers(0, 1 << 32, size=(2_000_003,), dtype=np.uint64).astype(np.uint32)
    a0 = a.copy()
    ta, tb = hip.from_numpy(a), hip.from_numpy(b)
    a[:] = 0  # the caller may reuse its memory as soon as the call returns
    np.testing.assert_array_equal(hip.to_numpy(tb), b)
    np.testing.assert_array_equal(hip.to_numpy(ta), a0)
